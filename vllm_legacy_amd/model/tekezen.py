"""Tekezen: a decoder-only stack over an fp32 stream whose sublayers read the stream itself and
are normed on their way out, with windowed softmax-attention layers and windowed latent-attention
layers in any order, dense or mixture-of-experts feed-forwards with a clamped gated activation,
and a hashed embedding of the (previous token, token) pair beside the token embedding.

  x = embed[token] + pair[(prev * mul_prev + token * mul_cur) mod buckets]   (row `buckets` for a
      sequence's first token)
  layer:  x <- x + N1(mixer(x));   x <- x + N2(ff(x))        (a layer may have no ff)
          N(u) = u / rms(u) * (1 + w)
  mixer 'attention':  q, k, v from x (kv_heads key / value heads for heads query heads); the whole
          q row and the whole k row RMS-normed with a weight per element; rotate-half rotary
          positions on the first rot.dims elements of a head, every frequency divided by
          rot.scaling.factor; score = (q . k) scale, capped by softcap tanh(score / softcap);
          position i sees j <= i with i - j < mask.size or j < mask.keep_first; softmax; in the
          layers marked v_mix but the first of them v <- (1 - lam) v + lam v_first, v_first that
          first layer's values of the same token (the blended v is what the cache holds); W_o
  mixer 'latent_attention':  q = W_q x (per head [plain | rotated]); W_dkv x = [latent | rotated
          key part], c = RMS norm of the latent; keys [W_uk c | k_rot], values W_uv c; rotate-half
          rotary positions with YaRN-scaled frequencies and magnitude on the rotated parts;
          score = (q . k) scale; position i sees 0 <= i - j < mask.size; softmax; head h's output
          times sigmoid(W_g x)_h; W_o
  ff 'dense':  W_down glu(W_gate x, W_up x),  glu(a, b) = g sigmoid(1.702 g) (u + 1) with
          g = min(a, limit), u = clamp(b, -limit, limit)
  ff 'moe':    the `top` largest router logits (W_r x, fp32) choose, the softmax over the chosen
          logits weighs, experts of the dense form; a shared expert of the same form (its own
          limit) is added for every token
  logits = embed N_final(x)

All sizes and per-model constants come from config.json; a layer entry carries its own mixer and
feed-forward sizes.  The projections that read x are one matrix product per sublayer; matrix
products go to the vendor library, everything else runs on libvla_seq_gfx950.so.  The stream,
norms, angles, attention scores and weights and routers are fp32 whatever `dtype` is; `dtype` is
the type of weights, projections, caches and activations (bfloat16 to serve, float32 for an
all-fp32 run).  Every update of the stream also leaves its copy in `dtype` for the next
projection, in the same launch.
"""
import json
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
from vllm_legacy_amd.attention.backends.rotary_kv import RotaryKVAttention
from vllm_legacy_amd.attention.batch import SequenceBatch
from vllm_legacy_amd.layers import GatedActivation, PairHashEmbedding
from vllm_legacy_amd.routed_experts import RoutedExperts, mm_f32

# constants of the gated activation that the design fixes
GLU_ALPHA = 1.702
GLU_SHIFT = 1.0


@dataclass
class AttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float              # 0: none
    window: int                 # 0: none
    keep_first: int
    rot_dims: int
    rot_base: float
    rot_factor: float           # every frequency is divided by it
    v_mix: bool


@dataclass
class LatentSpec:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int                 # 0: none
    rot_dims: int
    rot_base: float
    rot_scaling: Optional[Dict]


@dataclass
class MlpSpec:
    kind: str                   # dense | moe
    ff: int                     # dense: hidden size; moe: an expert's
    limit: float
    experts: int = 0
    top: int = 0
    shared_ff: int = 0
    shared_limit: float = 0.0


@dataclass
class LayerSpec:
    type: str                   # attention | latent_attention
    mixer: object
    mlp: Optional[MlpSpec]


@dataclass
class TekezenConfig:
    vocab: int
    width: int
    eps: float
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: List[LayerSpec]
    architecture: str = "Tekezen"
    raw: Dict = field(default_factory=dict, repr=False)

    @staticmethod
    def from_dict(d: Dict) -> "TekezenConfig":
        layers = []
        for i, entry in enumerate(d["layers"]):
            kind, m = entry.get("type"), entry.get("mixer") or {}
            rot, mask = m.get("rot") or {}, m.get("mask") or {}
            if kind == "attention":
                dim = int(m["dim"])
                mixer = AttentionSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), dim, int(m.get("vdim", dim)),
                                      float(m.get("scale", dim**-0.5)), float(m.get("softcap") or 0.0),
                                      int(mask.get("size") or 0), int(mask.get("keep_first") or 0),
                                      int(rot.get("dims", 0)), float(rot.get("base", 10000.0)),
                                      float((rot.get("scaling") or {}).get("factor", 1.0)), bool(m.get("v_mix", False)))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError(f"layer {i}: heads is not a multiple of kv_heads")
                if mixer.rot_dims % 2 or mixer.rot_dims > dim:
                    raise ValueError(f"layer {i}: rot.dims does not fit dim")
                if mixer.softcap < 0 or mixer.window < 0 or mixer.keep_first < 0 or mixer.rot_factor <= 0:
                    raise ValueError(f"layer {i}: softcap / mask / rot.scaling.factor out of range")
            elif kind == "latent_attention":
                dim, rot_dim = int(m["dim"]), int(m.get("rot_dim", 0))
                mixer = LatentSpec(int(m["heads"]), dim, rot_dim, int(m.get("vdim", dim)), int(m["kv_rank"]),
                                   float(m.get("scale", (dim + rot_dim)**-0.5)), int(mask.get("size") or 0),
                                   int(rot.get("dims", rot_dim)) if rot_dim else 0, float(rot.get("base", 10000.0)),
                                   rot.get("scaling") or None)
                if mixer.rot_dims % 2 or mixer.rot_dims > rot_dim:
                    raise ValueError(f"layer {i}: rot.dims does not fit rot_dim")
                if mixer.window < 0:
                    raise ValueError(f"layer {i}: mask.size out of range")
            else:
                raise ValueError(f"layer {i}: unknown layer type {kind!r}")
            mlp = entry.get("mlp")
            if mlp is None:
                spec = None
            elif mlp.get("kind") == "dense":
                spec = MlpSpec("dense", int(mlp["ff"]), float(mlp["limit"]))
            elif mlp.get("kind") == "moe":
                r, e, sh = mlp["router"], mlp["expert"], mlp.get("shared") or None
                spec = MlpSpec("moe", int(e["ff"]), float(e["limit"]), int(r["experts"]), int(r["top"]),
                               int(sh["ff"]) if sh else 0, float(sh["limit"]) if sh else 0.0)
                if spec.top < 1 or spec.top > spec.experts:
                    raise ValueError(f"layer {i}: router.top does not fit the number of experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            if spec is not None and (spec.limit <= 0 or (spec.shared_ff and spec.shared_limit <= 0)):
                raise ValueError(f"layer {i}: the activation's limit must be positive")
            layers.append(LayerSpec(kind, mixer, spec))
        mixed = [(s.mixer.kv_heads, s.mixer.vdim) for s in layers if s.type == "attention" and s.mixer.v_mix]
        if len(set(mixed)) > 1:
            raise ValueError("layers that blend their values must have the same kv_heads and vdim")
        bg = (d.get("embedding") or {}).get("bigram") or {}
        return TekezenConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), int(bg["buckets"]),
                             int(bg["mul_prev"]), int(bg["mul_cur"]), layers, d.get("architecture", "Tekezen"), d)

    @staticmethod
    def from_json(path: str) -> "TekezenConfig":
        with open(path) as f:
            return TekezenConfig.from_dict(json.load(f))


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


class TekezenLayer(nn.Module):

    def __init__(self, cfg: TekezenConfig, index: int, spec: LayerSpec, dtype, device):
        super().__init__()
        self.spec, self.dtype, self.eps, W = spec, dtype, cfg.eps, cfg.width

        def vec(n=W):
            return nn.Parameter(torch.ones(n, dtype=torch.float32, device=device), requires_grad=False)

        def mat(rows, cols, dt=dtype):
            return nn.Parameter(torch.zeros((rows, cols), dtype=dt, device=device), requires_grad=False)

        self.norm1 = vec()              # holds 1 + w
        m = spec.mixer
        if spec.type == "attention":
            self.attn = RotaryKVAttention(m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.rot_dims, m.rot_base,
                                          interleaved=False, window=m.window or None, device=device,
                                          keep_first=m.keep_first, softcap=m.softcap, freq_scale=m.rot_factor,
                                          norm_rows=True, norm_eps=cfg.eps)
            # the first layer that blends reads nobody's values: it is the one the others read
            prior = [s for s in cfg.layers[:index] if s.type == "attention" and s.mixer.v_mix]
            self.blends = m.v_mix and bool(prior)
            self.v_blend = nn.Parameter(torch.zeros(1, dtype=torch.float32, device=device),
                                        requires_grad=False) if m.v_mix else None
            self.in_names = ["mix.q", "mix.k", "mix.v"]
            self.in_widths = [m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim]
        else:
            self.attn = LatentKVAttention(m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, m.rot_dims,
                                          m.rot_base, m.rot_scaling, cfg.eps, dtype, device, interleaved=False,
                                          window=m.window or None)
            self.in_names = ["mix.q", "mix.dkv", "mix.g"]
            self.in_widths = [m.heads * (m.dim + m.rot_dim), m.kv_rank + m.rot_dim, m.heads]
        self.mixed = m.heads * m.vdim
        # every part of the merged input projection starts on a multiple of eight rows, so that each
        # part of a result row starts 16-byte aligned
        self.in_starts, rows = [], 0
        for n in self.in_widths:
            self.in_starts.append(rows)
            rows += _pad8(n)
        self.w_in = mat(rows, W)
        self.w_out = mat(W, self.mixed)
        mlp = spec.mlp
        if mlp is not None:
            self.norm2 = vec()
            if mlp.kind == "dense":
                self.w_gate_up, self.w_down = mat(2 * mlp.ff, W), mat(W, mlp.ff)
                self.act = GatedActivation("clamped_glu", True, mlp.limit, GLU_ALPHA, GLU_SHIFT)
            else:
                self.experts = RoutedExperts(W, mlp.experts, 0, mlp.top, mlp.ff, mlp.shared_ff, "clamped_glu",
                                             dtype=dtype, device=device, gated=True, act_limit=mlp.limit,
                                             act_alpha=GLU_ALPHA, act_shift=GLU_SHIFT, shared_gated=True,
                                             shared_limit=mlp.shared_limit)

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self, cfg: TekezenConfig) -> Dict[str, Tuple[int, ...]]:
        """Checkpoint names (without the layer prefix) and shapes of this layer's tensors."""
        W, m, mlp = cfg.width, self.spec.mixer, self.spec.mlp
        t: Dict[str, Tuple[int, ...]] = {"norm1": (W, )}
        for name, n in zip(self.in_names, self.in_widths):
            t[name] = (n, W)
        t["mix.o"] = (W, self.mixed)
        if self.spec.type == "attention":
            t.update({"mix.q.norm": (m.heads * m.dim, ), "mix.k.norm": (m.kv_heads * m.dim, )})
            if m.v_mix:
                t["mix.vmix"] = ()
        else:
            t.update({"mix.dkv.norm": (m.kv_rank, ), "mix.uk": (m.heads * m.dim, m.kv_rank),
                      "mix.uv": (m.heads * m.vdim, m.kv_rank)})
        if mlp is not None:
            t["norm2"] = (W, )
            if mlp.kind == "dense":
                t.update({"mlp.gate": (mlp.ff, W), "mlp.up": (mlp.ff, W), "mlp.down": (W, mlp.ff)})
            else:
                for e in range(mlp.experts):
                    t.update({f"mlp.e{e}.gate": (mlp.ff, W), f"mlp.e{e}.up": (mlp.ff, W), f"mlp.e{e}.down": (W, mlp.ff)})
                t["mlp.router"] = (mlp.experts, W)
                if mlp.shared_ff:
                    t.update({"mlp.shared.gate": (mlp.shared_ff, W), "mlp.shared.up": (mlp.shared_ff, W),
                              "mlp.shared.down": (W, mlp.shared_ff)})
        return t

    def set_weights(self, t: Dict[str, torch.Tensor], cfg: TekezenConfig) -> None:
        """t: this layer's tensors by their names without the layer prefix."""
        dev, dt, W = self.w_in.device, self.dtype, cfg.width
        for name, shape in self.tensor_shapes(cfg).items():
            if name not in t:
                raise KeyError(f"tensor {name} is missing")
            if tuple(t[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(t[name].shape)}, expected {shape}")

        def f32(name):
            return t[name].float().to(dev).contiguous()

        def put(param, value):
            param.data = value.to(param.dtype).to(dev).contiguous()

        self.norm1.data = 1.0 + f32("norm1")
        merged = torch.zeros(tuple(self.w_in.shape), dtype=dt)
        for name, n, start in zip(self.in_names, self.in_widths, self.in_starts):
            merged[start:start + n] = t[name].to(dt)
        put(self.w_in, merged)
        put(self.w_out, t["mix.o"])
        if self.spec.type == "attention":
            self.attn.q_norm.data, self.attn.k_norm.data = f32("mix.q.norm"), f32("mix.k.norm")
            if self.v_blend is not None:
                self.v_blend.data = f32("mix.vmix").reshape(1)
        else:
            self.attn.set_weights(t["mix.uk"], t["mix.uv"], t["mix.dkv.norm"])
        mlp = self.spec.mlp
        if mlp is not None:
            self.norm2.data = 1.0 + f32("norm2")
            if mlp.kind == "dense":
                put(self.w_gate_up, torch.cat([t["mlp.gate"], t["mlp.up"]], 0))
                put(self.w_down, t["mlp.down"])
            else:
                self.experts.set_weights({k[4:]: v for k, v in t.items() if k.startswith("mlp.")})

    # ------------------------------------------------------------------ caches
    def cache_shapes(self, cfg: TekezenConfig, num_blocks: int, block_size: int, num_slots: int):
        """name -> (shape, dtype) of what this layer keeps between steps."""
        m = self.spec.mixer
        if self.spec.type == "attention":
            ks, vs = RotaryKVAttention.get_cache_shapes(num_blocks, block_size, m.kv_heads, m.dim, m.vdim)
            return {"keys": (ks, self.dtype), "values": (vs, self.dtype)}
        return {"latent": (LatentKVAttention.get_cache_shape(num_blocks, block_size, m.kv_rank, m.rot_dim), self.dtype)}

    # ------------------------------------------------------------------ forward
    def _mix(self, h: torch.Tensor, batch: SequenceBatch, cache: Dict[str, torch.Tensor], shared: Dict) -> torch.Tensor:
        T, dev = h.shape[0], h.device
        proj = torch.mm(h, self.w_in.data.t())
        parts = [proj[:, s:s + n] for s, n in zip(self.in_starts, self.in_widths)]
        if self.spec.type == "attention":
            q, k, v = parts
            mixed = torch.empty((T, self.mixed), dtype=self.dtype, device=dev)
            if self.blends:
                self.attn(mixed, q, k, v, None, cache["keys"], cache["values"], batch, shared["v_first"],
                          self.v_blend.data)
            else:
                self.attn(mixed, q, k, v, None, cache["keys"], cache["values"], batch)
                if self.spec.mixer.v_mix:
                    shared["v_first"] = v       # a view of this step's projection; lives as long as the step
        else:
            q, kv, gate = parts
            mixed = self.attn(q, kv, cache["latent"], batch, gate)
        return mm_f32(mixed, self.w_out.data)

    def forward(self, x: torch.Tensor, h: torch.Tensor, batch: SequenceBatch, cache: Dict[str, torch.Tensor],
                shared: Dict) -> None:
        """x: fp32 [T, width], h: the same rows in the activation dtype; both updated in place."""
        ops.residual_norms(x, self._mix(h, batch, cache, shared), None, self.norm1.data, None, None, h, None, self.eps)
        mlp = self.spec.mlp
        if mlp is not None:
            if mlp.kind == "dense":
                y = mm_f32(self.act(torch.mm(h, self.w_gate_up.data.t())), self.w_down.data)
            else:
                y = self.experts(h)
            ops.residual_norms(x, y, None, self.norm2.data, None, None, h, None, self.eps)


class TekezenForCausalLM(nn.Module):
    """The stack and its per-layer caches.  `seed` fills random weights (benchmarks); load_weights
    installs a checkpoint's."""

    architecture = "Tekezen"

    def __init__(self, cfg: TekezenConfig, dtype=torch.bfloat16, device="cuda", seed: Optional[int] = None):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        W = cfg.width
        self.embed = PairHashEmbedding(cfg.vocab, W, cfg.buckets, cfg.mul_prev, cfg.mul_cur, dtype, device)
        self.layers = nn.ModuleList([TekezenLayer(cfg, i, s, dtype, device) for i, s in enumerate(cfg.layers)])
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32, device=device), requires_grad=False)
        if seed is not None:
            self.load_weights(self.random_weights(seed))

    # ------------------------------------------------------------------ caches
    def cache_spec(self) -> List[Dict[str, Tuple[int, ...]]]:
        """Per layer: the shapes of its caches for one block of one token; last, the embedding's
        state for one slot."""
        return [{k: v[0] for k, v in layer.cache_shapes(self.cfg, 1, 1, 1).items()} for layer in self.layers] + \
            [{"last_token": PairHashEmbedding.get_state_shape(1)}]

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int):
        """One entry per layer (its paged caches: a block id means the same block in each), then the
        embedding's state (a sequence's last token, by state slot)."""
        dev = self.final_norm.device
        caches = [{name: torch.zeros(shape, dtype=dt, device=dev)
                   for name, (shape, dt) in layer.cache_shapes(self.cfg, num_blocks, block_size, num_slots).items()}
                  for layer in self.layers]
        caches.append({"last_token": torch.zeros(PairHashEmbedding.get_state_shape(num_slots), dtype=torch.int64,
                                                 device=dev)})
        return caches

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, caches, batch: SequenceBatch,
                tap=None) -> torch.Tensor:
        """Returns the fp32 stream [T, width] after the last layer.  tap(layer, x) is called after
        every layer (tests, layer-by-layer comparison)."""
        x = self.embed(input_ids, caches[len(self.layers)]["last_token"], batch)
        h = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        ops.residual_norms(x, out=h)
        shared: Dict = {}
        for i, layer in enumerate(self.layers):
            layer(x, h, batch, caches[i], shared)
            if tap is not None:
                tap(i, x)
        return x

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """hidden: the rows of the stream whose logits are wanted -> fp32 [n, vocab]."""
        x = hidden.contiguous()
        h = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        ops.residual_norms(x, out=h, pre_weight=self.final_norm.data, eps=self.cfg.eps)
        return mm_f32(h, self.embed.weight.data)

    # ------------------------------------------------------------------ weights
    def _top_shapes(self) -> Dict[str, Tuple[int, ...]]:
        cfg = self.cfg
        return {"embed": (cfg.vocab, cfg.width), "bigram": (cfg.buckets + 1, cfg.width), "final.norm": (cfg.width, )}

    def tensor_shapes(self) -> Dict[str, Tuple[int, ...]]:
        t = self._top_shapes()
        for i, layer in enumerate(self.layers):
            t.update({f"l{i}.{k}": v for k, v in layer.tensor_shapes(self.cfg).items()})
        return t

    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> int:
        cfg, dev = self.cfg, self.final_norm.device
        used = 0
        for i, layer in enumerate(self.layers):
            prefix = f"l{i}."
            mine = {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
            layer.set_weights(mine, cfg)
            used += len(layer.tensor_shapes(cfg))
        top = self._top_shapes()
        for name, shape in top.items():
            if name not in tensors:
                raise KeyError(f"tensor {name} is missing")
            if tuple(tensors[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}, expected {shape}")
        self.embed.weight.data = tensors["embed"].to(self.dtype).to(dev).contiguous()
        self.embed.pair_weight.data = tensors["bigram"].to(self.dtype).to(dev).contiguous()
        self.final_norm.data = 1.0 + tensors["final.norm"].float().to(dev).contiguous()
        return used + len(top)

    def random_weights(self, seed: int) -> Dict[str, torch.Tensor]:
        """Tensors of every checkpoint name: projections ~ N(0, 1 / fan_in), norm weights of the
        stream near 0 (they are stored around zero), the query / key norms' near 1, blends in
        (0, 1)."""
        g = torch.Generator().manual_seed(seed)
        out = {}
        for name, shape in self.tensor_shapes().items():
            last = name.rsplit(".", 1)[-1]
            if name in ("embed", "bigram"):
                t = torch.randn(shape, generator=g)
            elif last == "vmix":
                t = 0.2 + 0.6 * torch.rand(shape, generator=g)
            elif last in ("norm1", "norm2") or name == "final.norm":
                t = 0.1 * torch.randn(shape, generator=g)
            elif last == "norm":
                t = 1.0 + 0.1 * torch.randn(shape, generator=g)
            else:
                t = torch.randn(shape, generator=g) * shape[-1]**-0.5
            out[name] = t.to(torch.bfloat16)
        return out
