"""Slow reference of the Lamosun design in float64 on the CPU, one function per mechanism, written
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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms_norm(u, w, eps):
    """u / sqrt(mean(u^2) + eps) * w over the last axis."""
    return u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * w


def short_convolution(u, w, bias=None):
    """u [n, C], w [C, taps]: out_t = sum_j w[:, j] u_(t - taps + 1 + j) (+ bias), zeros before the
    start; the last column weighs the current token."""
    n, taps = u.shape[0], w.shape[1]
    out = torch.zeros_like(u)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * u[s]
    return out if bias is None else out + bias


# ----------------------------------------------------------------------------- gated delta rule
def delta_rule(q, k, v, beta, decay, S=None):
    """One head: q, k [n, D] (normed already), v [n, V], beta, decay [n].  S <- decay S;
    u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Returns o [n, V] (and leaves S updated)."""
    n, D, V = q.shape[0], q.shape[1], v.shape[1]
    if S is None:
        S = torch.zeros(D, V, dtype=F)
    out = torch.zeros(n, V, dtype=F)
    for i in range(n):
        S *= decay[i]
        u = beta[i] * (v[i] - S.T @ k[i])
        S += torch.outer(k[i], u)
        out[i] = S.T @ q[i]
    return out


def delta_mixer(h, t, spec, eps):
    """h [n, W]; t: the mixer's tensors by their short names; spec: heads, kv_heads, dim, vdim."""
    n = h.shape[0]
    H, G, D, V = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    q = silu(short_convolution(h @ t["q"].T, t["q.conv"])).view(n, G, D)
    k = silu(short_convolution(h @ t["k"].T, t["k.conv"])).view(n, G, D)
    v = silu(short_convolution(h @ t["v"].T, t["v.conv"])).view(n, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D**-0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ t["b"].T)                                          # [n, H]
    decay = torch.exp(-torch.exp(t["A_log"]) * softplus(h @ t["a"].T + t["dt_bias"]))
    gate = silu(h @ t["g"].T).view(n, H, V)
    out = torch.zeros(n, H, V, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        out[:, hh] = delta_rule(q[:, g], k[:, g], v[:, hh], beta[:, hh], decay[:, hh])
    out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps) * t["norm"] * gate
    return out.reshape(n, H * V) @ t["o"].T


# ----------------------------------------------------------------------------- real-gated LRU
def rglru_recurrence(u, r, i, lam, S=None):
    """u, r, i [n, R] (gates after their sigmoid), lam [R]: a = exp(-8 r softplus(lam)),
    S_t = a S_(t-1) + sqrt(1 - a^2) i u from S = 0.  Returns every S_t."""
    a = torch.exp(-8.0 * r * softplus(lam))
    S = torch.zeros(u.shape[1], dtype=F) if S is None else S
    out = torch.zeros_like(u)
    for s_ in range(u.shape[0]):
        S = a[s_] * S + torch.sqrt(1.0 - a[s_]**2) * i[s_] * u[s_]
        out[s_] = S
    return out


def rglru_mixer(h, t, spec):
    """h [n, W]; spec: width, blocks."""
    n = h.shape[0]
    R, B = spec["width"], spec["blocks"]
    y = gelu_tanh(h @ t["y"].T + t["y.b"])
    u = short_convolution(h @ t["x"].T + t["x.b"], t["conv"], t["conv.b"])
    ub = u.view(n, B, R // B)
    r = torch.sigmoid(torch.einsum("boi,nbi->nbo", t["ra"], ub) + t["ra.b"]).reshape(n, R)
    i = torch.sigmoid(torch.einsum("boi,nbi->nbo", t["ri"], ub) + t["ri.b"]).reshape(n, R)
    out = rglru_recurrence(u, r, i, t["lam"])
    return (out * y) @ t["o"].T


# ----------------------------------------------------------------------------- latent attention
def yarn_frequencies(rot):
    """Per pair: the frequency after scaling, and the factor on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F)
    f = torch.pow(torch.tensor(float(base), dtype=F), -2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def where(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    return f / sc["factor"] * ramp + f * (1 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_interleaved(u, positions, rot):
    """u [n, heads, dims]: pair (2i, 2i + 1) at position p turned by p * f_i."""
    f, mag = yarn_frequencies(rot)
    ang = (positions.to(torch.float32)[:, None] * f.to(torch.float32)[None, :]).to(F)
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = u[..., 0::2], u[..., 1::2]
    out = torch.empty_like(u)
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = b * c + a * s
    return out


def latent_attention_mixer(h, t, spec, eps):
    """h [n, W]; spec: heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot."""
    n = h.shape[0]
    H, D, Rr, V, C = spec["heads"], spec["dim"], spec["rot_dim"], spec["vdim"], spec["kv_rank"]
    pos = torch.arange(n)
    q = (rms_norm(h @ t["dq"].T, t["dq.norm"], eps) @ t["uq"].T).view(n, H, D + Rr)
    kv = h @ t["dkv"].T
    c = rms_norm(kv[:, :C], t["dkv.norm"], eps)
    k_rot = rotate_interleaved(kv[:, None, C:], pos, spec["rot"])[:, 0]            # [n, Rr]
    q_plain, q_rot = q[..., :D], rotate_interleaved(q[..., D:], pos, spec["rot"])
    k_plain = (c @ t["uk"].T).view(n, H, D)
    v = (c @ t["uv"].T).view(n, H, V)
    out = torch.zeros(n, H, V, dtype=F)
    for a in range(n):
        for hh in range(H):
            s = (k_plain[:a + 1, hh] @ q_plain[a, hh] + k_rot[:a + 1] @ q_rot[a, hh]) * spec["scale"]
            out[a, hh] = torch.softmax(s, 0) @ v[:a + 1, hh]
    return out.reshape(n, H * V) @ t["o"].T


# ----------------------------------------------------------------------------- feed-forwards
def dense_ff(h, t):
    return (gelu_tanh(h @ t["gate"].T) * (h @ t["up"].T)) @ t["down"].T


def routed_ff(h, t, spec):
    """spec: router.experts, router.top."""
    E, top = spec["router"]["experts"], spec["router"]["top"]
    z = h @ t["router"].T + t["router.b"]
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        val, idx = torch.topk(z[i], top)
        w = torch.softmax(val, 0)
        for j in range(top):
            e = int(idx[j])
            g, u, d = t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"]
            out[i] += w[j] * ((silu(g @ h[i]) * (u @ h[i])) @ d.T)
    assert E == z.shape[1]
    return out


def token_side_input(x, e, t, eps):
    """x [n, W], e [n, dim] the layer's part of the tokens' side embedding."""
    y = (gelu_tanh(x @ t["gate"].T) * e) @ t["proj"].T
    return x + y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * t["norm"]


# ----------------------------------------------------------------------------- the model
def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F) for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, layer_out=None):
    """tokens: a list of ids of one sequence.  Returns logits [n, vocab] (float64); layer_out, a
    list, receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    alpha = cfg.get("postln_alpha", 1.0)
    ids = torch.as_tensor(tokens, dtype=torch.int64)
    x = tensors["embed"].to(F)[ids] * (cfg.get("embedding") or {}).get("scale", 1.0)
    side = cfg.get("token_side")
    for i, layer in enumerate(cfg["layers"]):
        t = sub(tensors, f"l{i}.mix.")
        kind = layer["type"]
        if kind == "delta":
            y = delta_mixer(x, t, layer["mixer"], eps)
        elif kind == "rglru":
            y = rglru_mixer(x, t, layer["mixer"])
        elif kind == "latent_attention":
            y = latent_attention_mixer(x, t, layer["mixer"], eps)
        else:
            raise ValueError(kind)
        x = rms_norm(alpha * x + y, tensors[f"l{i}.norm1"].to(F), eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            t = sub(tensors, f"l{i}.mlp.")
            y = dense_ff(x, t) if mlp["kind"] == "dense" else routed_ff(x, t, mlp)
            x = rms_norm(alpha * x + y, tensors[f"l{i}.norm2"].to(F), eps)
        if side:
            d = side["dim"]
            e = tensors["side.embed"].to(F)[ids][:, i * d:(i + 1) * d]
            x = token_side_input(x, e, sub(tensors, f"l{i}.side."), eps)
        if layer_out is not None:
            layer_out.append(x.clone())
    x = rms_norm(x, tensors["final.norm"].to(F), eps)
    logits = x @ tensors["head"].to(F).T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits


def latent_attention_core(q_lat, q_rot, c, k_rot, scale, first=0):
    """q_lat [n, H, C], q_rot [n, H, R] for the positions first .. first + n - 1; c [m, C], k_rot
    [m, R] every position from 0.  Returns sum_j p_j c_j [n, H, C], p the causal softmax of
    (q_lat . c_j + q_rot . k_rot_j) * scale."""
    n, H, C = q_lat.shape
    out = torch.zeros(n, H, C, dtype=F)
    for a in range(n):
        m = first + a + 1
        for hh in range(H):
            s = (c[:m] @ q_lat[a, hh] + k_rot[:m] @ q_rot[a, hh]) * scale
            out[a, hh] = torch.softmax(s, 0) @ c[:m]
    return out


def spread(logits):
    """Root mean square of the logits around their mean over the vocabulary, averaged over rows."""
    c = logits - logits.mean(-1, keepdim=True)
    return float(torch.sqrt((c * c).mean(-1)).mean())


def row_errors(got, want):
    """Per row: rms over the vocabulary of the difference with its mean taken off."""
    d = got.to(F) - want.to(F)
    d = d - d.mean(-1, keepdim=True)
    return torch.sqrt((d * d).mean(-1))


# ----------------------------------------------------------------------------- small random models
def delta_layer(heads, kv_heads, dim, vdim=None, conv=4, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim or dim, "conv": conv},
            "mlp": mlp}


def rglru_layer(width, blocks, conv=4, mlp=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": mlp}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale=None, base=10000.0, scaling=None, mlp=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "scale": (dim + rot_dim)**-0.5 if scale is None else scale,
                      "rot": {"base": base, "dims": rot_dim, **({"scaling": scaling} if scaling else {})}},
            "mlp": mlp}


def dense_mlp(ff):
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_config(layers, vocab=97, width=64, eps=1e-5, alpha=1.5, embed_scale=3.0, side_dim=8, softcap=20.0):
    cfg = {"architecture": "Lamosun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
           "embedding": {"scale": embed_scale}, "layers": layers}
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
    if softcap:
        cfg["logit_softcap"] = softcap
    return cfg


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    L = len(cfg["layers"])
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W, )}
    side = cfg.get("token_side")
    if side:
        out["side.embed"] = (V, L * side["dim"])
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W, )
        if layer["type"] == "delta":
            H, G, D, Vd, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            out.update({p + "mix.q": (G * D, W), p + "mix.q.conv": (G * D, taps), p + "mix.k": (G * D, W),
                        p + "mix.k.conv": (G * D, taps), p + "mix.v": (H * Vd, W), p + "mix.v.conv": (H * Vd, taps),
                        p + "mix.b": (H, W), p + "mix.A_log": (H, ), p + "mix.norm": (Vd, ), p + "mix.a": (H, W),
                        p + "mix.dt_bias": (H, ), p + "mix.g": (H * Vd, W), p + "mix.o": (W, H * Vd)})
        elif layer["type"] == "rglru":
            R, B, taps = m["width"], m["blocks"], m["conv"]
            out.update({p + "mix.y": (R, W), p + "mix.y.b": (R, ), p + "mix.x": (R, W), p + "mix.x.b": (R, ),
                        p + "mix.conv": (R, taps), p + "mix.conv.b": (R, ), p + "mix.ra": (B, R // B, R // B),
                        p + "mix.ra.b": (B, R // B), p + "mix.ri": (B, R // B, R // B), p + "mix.ri.b": (B, R // B),
                        p + "mix.lam": (R, ), p + "mix.o": (W, R)})
        else:
            H, D, Rr, Vd, C, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({p + "mix.dq": (Q, W), p + "mix.dq.norm": (Q, ), p + "mix.uq": (H * (D + Rr), Q),
                        p + "mix.dkv": (C + Rr, W), p + "mix.dkv.norm": (C, ), p + "mix.uk": (H * D, C),
                        p + "mix.uv": (H * Vd, C), p + "mix.o": (W, H * Vd)})
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
                out[p + "mlp.router.b"] = (mlp["router"]["experts"], )
        if side:
            out.update({p + "side.gate": (side["dim"], W), p + "side.proj": (W, side["dim"]), p + "side.norm": (W, )})
    return out


def random_tensors(cfg, seed):
    """bfloat16 tensors of every checkpoint name: projections ~ N(0, 1 / fan_in), norm weights near
    1, biases and convolution taps of moderate size."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name in ("embed", "side.embed"):
            t = torch.randn(shape, generator=g)
        elif last == "norm" or name.endswith("norm1") or name.endswith("norm2"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last in ("A_log", "dt_bias", "lam", "b") and len(shape) <= 2 and not name.endswith("mix.b"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif last in ("ra", "ri"):
            t = torch.randn(shape, generator=g) * shape[-1]**-0.5
        else:
            t = torch.randn(shape, generator=g) * shape[-1]**-0.5
            if ".mix." in name and last in ("q", "k", "v", "x", "uq", "dkv", "b", "a"):
                t = t * 2.0
        out[name] = t.to(torch.bfloat16)
    return out


def write_checkpoint(folder, cfg, tensors):
    """config.json + model.safetensors (bfloat16 / int32 data, names sorted)."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name in sorted(tensors):
        t = tensors[name].contiguous()
        code = {torch.bfloat16: "BF16", torch.float32: "F32", torch.int32: "I32"}[t.dtype]
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
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
