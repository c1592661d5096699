"""Slow reference of the Tekezen design in float64 on the CPU, one function per mechanism, written
from the equations and sharing no code with vllm_legacy_amd.  Also the helpers that make small
random models (config dict + tensors under their checkpoint names) and write them as a
checkpoint folder.

Notation: x[t] the stream at token t (position t, counted from 0 in its sequence), W y a linear
map stored [out, in].  Every function takes one whole sequence from its first token.
"""
import json
import math
import os
import struct

import torch

F = torch.float64
GLU_ALPHA, GLU_SHIFT = 1.702, 1.0


def rms_norm(u, w, eps):
    """u / sqrt(mean(u^2) + eps) * w over the last axis."""
    return u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * w


def stream_norm(u, w, eps):
    """The norm of a sublayer's output: its weight is stored around zero."""
    return rms_norm(u, 1.0 + w, eps)


def clamped_glu(a, b, limit):
    """g sigmoid(1.702 g) (u + 1) with g = min(a, limit), u = clamp(b, -limit, limit)."""
    g = torch.minimum(a, torch.tensor(limit, dtype=F))
    u = torch.clamp(b, -limit, limit)
    return g * torch.sigmoid(GLU_ALPHA * g) * (u + GLU_SHIFT)


# ----------------------------------------------------------------------------- embedding
def pair_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table per token: a hash of (previous token, token); the table's last row
    (number `buckets`) for the first token."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((prev * mul_prev + cur * mul_cur) % buckets)
    return rows


def embedding(tokens, embed, pair, bigram):
    rows = pair_rows(list(tokens), bigram["buckets"], bigram["mul_prev"], bigram["mul_cur"])
    return embed[torch.tensor(list(tokens))] + pair[torch.tensor(rows)]


# ----------------------------------------------------------------------------- rotary positions
def plain_frequencies(dims, base):
    i = torch.arange(dims // 2, dtype=F)
    return float(base)**(-2.0 * i / dims)


def yarn_frequencies(rot):
    """(frequencies [dims / 2], magnitude) for rot = {dims, base, scaling: {factor, original, fast,
    slow}} (no scaling: plain frequencies, magnitude 1)."""
    dims, base, sc = rot["dims"], float(rot["base"]), rot.get("scaling")
    f = plain_frequencies(dims, base)
    if not sc:
        return f, 1.0
    i = torch.arange(dims // 2, dtype=F)

    def where(turns):       # the pair that makes `turns` turns over the original length
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half(u, positions, freqs, magnitude=1.0):
    """u [n, heads, d]: element i < len(freqs) pairs with element i + len(freqs); the pair (a, b) at
    position p becomes (a cos - b sin, b cos + a sin) of p f_i, sine and cosine times magnitude;
    elements from 2 len(freqs) on pass unchanged."""
    half = freqs.numel()
    ang = positions.to(F)[:, None] * freqs[None, :]
    c, s = (torch.cos(ang) * magnitude)[:, None, :], (torch.sin(ang) * magnitude)[:, None, :]
    a, b = u[..., :half], u[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, u[..., 2 * half:]], -1)


# ----------------------------------------------------------------------------- attention
def visible(n, window, keep_first=0, first=0):
    """[n - first, n] bool: query i (from `first` on) sees key j <= i with i - j < window or
    j < keep_first (window 0: every j <= i)."""
    i = torch.arange(first, n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if window:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def attention_core(q, k, v, scale, softcap=0.0, window=0, keep_first=0, first=0):
    """q [m, H, D] (queries of positions first ..), k [n, G, D], v [n, G, V] -> [m, H, V]."""
    H, G = q.shape[1], k.shape[1]
    kk, vv = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    s = s.masked_fill(~visible(k.shape[0], window, keep_first, first), -math.inf)
    return torch.einsum("hij,jhv->ihv", torch.softmax(s, -1), vv)


def attention_mixer(h, t, spec, eps, v_first=None):
    """t: the mixer's tensors (q, k, v, q.norm, k.norm, vmix, o).  Returns (output, the values
    before any blend)."""
    n = h.shape[0]
    H, G, D, V = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    pos = torch.arange(n)
    rot, mask = spec["rot"], spec.get("mask") or {}
    f = plain_frequencies(rot["dims"], rot["base"]) / (rot.get("scaling") or {}).get("factor", 1.0)
    q = rotate_half(rms_norm(h @ t["q"].T, t["q.norm"], eps).view(n, H, D), pos, f)
    k = rotate_half(rms_norm(h @ t["k"].T, t["k.norm"], eps).view(n, G, D), pos, f)
    v_own = h @ t["v"].T
    v = v_own if v_first is None else (1.0 - t["vmix"]) * v_own + t["vmix"] * v_first
    o = attention_core(q, k, v.view(n, G, V), spec["scale"], spec.get("softcap") or 0.0, mask.get("size") or 0,
                       mask.get("keep_first") or 0)
    return o.reshape(n, H * V) @ t["o"].T, v_own


def latent_attention_mixer(h, t, spec, eps):
    """t: q, dkv, dkv.norm, uk, uv, g, o."""
    n = h.shape[0]
    H, D, Rr, V, C = spec["heads"], spec["dim"], spec["rot_dim"], spec["vdim"], spec["kv_rank"]
    pos = torch.arange(n)
    f, mag = yarn_frequencies(spec["rot"]) if Rr else (torch.zeros(0, dtype=F), 1.0)
    q = (h @ t["q"].T).view(n, H, D + Rr)
    down = h @ t["dkv"].T
    c = rms_norm(down[:, :C], t["dkv.norm"], eps)
    k_rot = rotate_half(down[:, C:].view(n, 1, Rr), pos, f, mag)
    q_rot = rotate_half(q[..., D:], pos, f, mag)
    k = torch.cat([(c @ t["uk"].T).view(n, H, D), k_rot.expand(n, H, Rr)], -1)
    v = (c @ t["uv"].T).view(n, H, V)
    o = attention_core(torch.cat([q[..., :D], q_rot], -1), k, v, spec["scale"], 0.0, (spec.get("mask") or {}).get("size") or 0)
    gate = torch.sigmoid(h @ t["g"].T)
    return (o * gate[:, :, None]).reshape(n, H * V) @ t["o"].T


def latent_attention_core(q_lat, q_rot, c, k_rot, scale, window=0, first=0, gate=None):
    """The latent-side form: q_lat [m, H, C], q_rot [m, H, R] (rotated), c [n, C], k_rot [n, R]
    (rotated) -> sum_j p_j c_j [m, H, C] (times sigmoid(gate [m, H]))."""
    s = (torch.einsum("ihc,jc->hij", q_lat, c) + torch.einsum("ihr,jr->hij", q_rot, k_rot)) * scale
    s = s.masked_fill(~visible(c.shape[0], window, 0, first), -math.inf)
    o = torch.einsum("hij,jc->ihc", torch.softmax(s, -1), c)
    return o if gate is None else o * torch.sigmoid(gate)[:, :, None]


# ----------------------------------------------------------------------------- feed-forwards
def dense_ff(h, t, limit):
    return clamped_glu(h @ t["gate"].T, h @ t["up"].T, limit) @ t["down"].T


def routed_ff(h, t, spec):
    """The `top` largest router logits choose; the softmax over the chosen logits weighs; a shared
    expert, when there is one, is added for every token."""
    z = h @ t["router"].T
    val, idx = torch.topk(z, spec["router"]["top"], dim=-1)
    wt = torch.softmax(val, -1)
    out = torch.zeros(h.shape[0], t["e0.down"].shape[0], dtype=F)
    for i in range(h.shape[0]):
        for kx in range(idx.shape[1]):
            e = int(idx[i, kx])
            out[i] += wt[i, kx] * dense_ff(h[i:i + 1], sub(t, f"e{e}."), spec["expert"]["limit"])[0]
    if spec.get("shared"):
        out = out + dense_ff(h, sub(t, "shared."), spec["shared"]["limit"])
    return out


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, layer_out=None):
    """Logits [n, vocab] of one sequence; layer_out (a list) receives the stream after every layer."""
    t = {k: v.to(F) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x = embedding(tokens, t["embed"], t["bigram"], cfg["embedding"]["bigram"])
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        lt = sub(t, f"l{i}.")
        if layer["type"] == "attention":
            blends = layer["mixer"].get("v_mix")
            y, v_own = attention_mixer(x, sub(lt, "mix."), layer["mixer"], eps, v_first if blends else None)
            if blends and v_first is None:
                v_first = v_own
        else:
            y = latent_attention_mixer(x, sub(lt, "mix."), layer["mixer"], eps)
        x = x + stream_norm(y, lt["norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            y = dense_ff(x, sub(lt, "mlp."), mlp["limit"]) if mlp["kind"] == "dense" else routed_ff(x, sub(lt, "mlp."), mlp)
            x = x + stream_norm(y, lt["norm2"], eps)
        if layer_out is not None:
            layer_out.append(x.clone())
    return stream_norm(x, t["final.norm"], eps) @ t["embed"].T


def spread(logits):
    """Root mean square over a request of the logits with each row's mean taken off."""
    d = logits - logits.mean(-1, keepdim=True)
    return torch.sqrt((d * d).mean())


def row_errors(got, want):
    """Per row: rms over the vocabulary of the difference with its mean taken off."""
    d = got.to(F) - want.to(F)
    d = d - d.mean(-1, keepdim=True)
    return torch.sqrt((d * d).mean(-1))


# ----------------------------------------------------------------------------- small random models
def attention_layer(heads, kv_heads, dim, vdim=None, window=0, keep_first=0, rot_dims=None, base=10000.0, factor=None,
                    scale=None, softcap=None, v_mix=False, mlp=None):
    rot = {"base": base, "dims": dim if rot_dims is None else rot_dims}
    if factor:
        rot["scaling"] = {"factor": factor}
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim or dim, "rot": rot,
         "scale": dim**-0.5 if scale is None else scale}
    if window:
        m["mask"] = {"size": window, "keep_first": keep_first}
    if softcap:
        m["softcap"] = softcap
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, window=0, scale=None, base=10000.0, scaling=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": (dim + rot_dim)**-0.5 if scale is None else scale,
         "rot": {"base": base, "dims": rot_dim, **({"scaling": scaling} if scaling else {})}}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense_mlp(ff, limit=2.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe_mlp(experts, top, ff, limit=2.0, shared_ff=0, shared_limit=1.0):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared_ff:
        out["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return out


def make_config(layers, vocab=97, width=64, eps=1e-5, buckets=53, mul_prev=13, mul_cur=5):
    return {"architecture": "Tekezen", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}, "layers": layers}


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "bigram": (cfg["embedding"]["bigram"]["buckets"] + 1, W), "final.norm": (W, )}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W, )
        if layer["type"] == "attention":
            H, G, D, Vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, W), p + "mix.k": (G * D, W), p + "mix.v": (G * Vd, W),
                        p + "mix.q.norm": (H * D, ), p + "mix.k.norm": (G * D, ), p + "mix.o": (W, H * Vd)})
            if m.get("v_mix"):
                out[p + "mix.vmix"] = ()
        else:
            H, D, Rr, Vd, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            out.update({p + "mix.q": (H * (D + Rr), W), p + "mix.dkv": (C + Rr, W), p + "mix.dkv.norm": (C, ),
                        p + "mix.uk": (H * D, C), p + "mix.uv": (H * Vd, C), p + "mix.g": (H, W), p + "mix.o": (W, H * Vd)})
        mlp = layer.get("mlp")
        if mlp is not None:
            out[p + "norm2"] = (W, )
            if mlp["kind"] == "dense":
                out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
            else:
                ff = mlp["expert"]["ff"]
                for e in range(mlp["router"]["experts"]):
                    out.update({p + f"mlp.e{e}.gate": (ff, W), p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
                out[p + "mlp.router"] = (mlp["router"]["experts"], W)
                if mlp.get("shared"):
                    sf = mlp["shared"]["ff"]
                    out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W), p + "mlp.shared.down": (W, sf)})
    return out


def random_tensors(cfg, seed):
    """bfloat16 tensors of every checkpoint name: projections ~ N(0, 1 / fan_in) (those of queries,
    keys and feed-forward inputs larger, so that scores spread and the activation's clamps bite),
    stream norm weights around 0, query / key / latent norm weights around 1, blends in (0, 1)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name in ("embed", "bigram"):
            t = torch.randn(shape, generator=g)
        elif last in ("norm1", "norm2") or name == "final.norm":
            t = 0.2 * torch.randn(shape, generator=g)
        elif last == "norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "vmix":
            t = 0.2 + 0.6 * torch.rand(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * shape[-1]**-0.5
            if last in ("q", "k", "dkv", "gate", "up", "g"):
                t = t * 2.0
        out[name] = t.to(torch.bfloat16)
    return out


def write_checkpoint(folder, cfg, tensors):
    """config.json + model.safetensors (bfloat16 data, names sorted)."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name in sorted(tensors):
        t = tensors[name].contiguous()
        code = {torch.bfloat16: "BF16", torch.float32: "F32", torch.int32: "I32"}[t.dtype]
        raw = t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": code, "shape": list(t.shape), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    hj = json.dumps(header).encode()
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)
    return folder
