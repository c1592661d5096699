"""Lamosun: a decoder-only stack over an fp32 stream that is normed after every sublayer, with
gated-delta-rule layers, real-gated linear recurrent layers and latent-attention layers in any
order, dense or mixture-of-experts feed-forwards, and a per-layer input from a side embedding of the
token.

  x = embed[token] * scale
  layer:  x <- N1(alpha x + mixer(x));   x <- N2(alpha x + ff(x))   (a layer may have no ff)
          N(u) = u / rms(u) * w; the sublayers read x itself
          side input (when the model has one): e = the layer's columns of side.embed[token],
          y = W_proj (gelu_tanh(W_gate x) * e),  x <- x + y / rms(y) * w_side
  mixer 'delta':  q, k (kv_heads x dim), v (heads x vdim) from x, each through a short causal
          convolution and silu; q, k unit vectors per head, q times dim^-1/2; beta = sigmoid(W_b x),
          g = exp(-exp(A_log) softplus(W_a x + dt_bias)); per head S <- g S, u = beta (v - S^T k),
          S <- S + k u^T, o = S^T q; o / rms(o) * w * silu(W_g x), then W_o
  mixer 'rglru':  y = gelu_tanh(W_y x + b), u = conv(W_x x + b) + b_conv; block-diagonal gates
          r = sigmoid(W_a u + b), i = sigmoid(W_i u + b); a = exp(-8 r softplus(lam));
          S <- a S + sqrt(1 - a^2) i u; W_o (S * y)
  mixer 'latent_attention':  c_q = N(W_dq x), q = W_uq c_q (per head [plain | rotated]);
          W_dkv x = [latent | rotated key part], c = N(latent); keys [W_uk c | k_rot], values W_uv c;
          rotary positions (YaRN-scaled frequencies) on the rotated parts; causal softmax; W_o
  ff 'dense':  W_down (gelu_tanh(W_gate x) * W_up x)
  ff 'moe':    top experts by router logits (W_r x + b, fp32), weights = softmax over the chosen
          logits, experts W_down (silu(W_gate x) * W_up x)
  logits = cap * tanh(head N_final(x) / cap)

All sizes and per-model constants come from config.json; a layer entry carries its own mixer and
feed-forward sizes.  The projections that read x are one matrix product per sublayer; matrix
products go to the vendor library, everything else runs on libvla_seq_gfx950.so.  The stream,
norms, angles, attention scores and weights, routers, everything that enters a recurrence and its
state are fp32 whatever `dtype` is; `dtype` is the type of weights, projections and activations
(bfloat16 to serve, float32 for an all-fp32 run).  Every update of the stream also leaves its copy
in `dtype` for the next projection, in the same launch.
"""
import json
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.backends.latent_kv import LatentKVAttention
from vllm_legacy_amd.attention.batch import SequenceBatch
from vllm_legacy_amd.attention.recurrent import GatedDeltaRule, RealGatedLRU
from vllm_legacy_amd.layers import GatedActivation, ShortConv, TokenGatedInput
from vllm_legacy_amd.routed_experts import RoutedExperts, mm_f32


@dataclass
class DeltaSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    taps: int


@dataclass
class RGLRUSpec:
    width: int
    blocks: int
    taps: int


@dataclass
class LatentAttentionSpec:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_dims: int
    rot_base: float
    rot_scaling: Optional[Dict]


@dataclass
class MlpSpec:
    kind: str                   # dense | moe
    ff: int                     # dense: hidden size; moe: an expert's
    experts: int = 0
    top: int = 0


@dataclass
class LayerSpec:
    type: str                   # delta | rglru | latent_attention
    mixer: object
    mlp: Optional[MlpSpec]


@dataclass
class LamosunConfig:
    vocab: int
    width: int
    eps: float
    alpha: float
    embed_scale: float
    side_dim: int               # 0: no side input
    softcap: float              # 0: none
    layers: List[LayerSpec]
    architecture: str = "Lamosun"
    raw: Dict = field(default_factory=dict, repr=False)

    @staticmethod
    def from_dict(d: Dict) -> "LamosunConfig":
        layers = []
        for i, entry in enumerate(d["layers"]):
            kind, m = entry.get("type"), entry.get("mixer") or {}
            if kind == "delta":
                mixer = DeltaSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]),
                                  int(m.get("vdim", m["dim"])), int(m.get("conv", 1)))
                if mixer.heads % mixer.kv_heads or mixer.taps < 1:
                    raise ValueError(f"layer {i}: heads / kv_heads / conv do not fit")
            elif kind == "rglru":
                mixer = RGLRUSpec(int(m["width"]), int(m.get("blocks", 1)), int(m.get("conv", 1)))
                if mixer.width % mixer.blocks or mixer.taps < 1:
                    raise ValueError(f"layer {i}: width / blocks / conv do not fit")
            elif kind == "latent_attention":
                rot = m.get("rot") or {}
                dim, rot_dim = int(m["dim"]), int(m.get("rot_dim", 0))
                mixer = LatentAttentionSpec(int(m["heads"]), dim, rot_dim, int(m.get("vdim", dim)), int(m["kv_rank"]),
                                            int(m["q_rank"]), float(m.get("scale", (dim + rot_dim)**-0.5)),
                                            int(rot.get("dims", rot_dim)) if rot_dim else 0,
                                            float(rot.get("base", 10000.0)), rot.get("scaling") or None)
                if mixer.rot_dims % 2 or mixer.rot_dims > rot_dim:
                    raise ValueError(f"layer {i}: rot.dims does not fit rot_dim")
            else:
                raise ValueError(f"layer {i}: unknown layer type {kind!r}")
            mlp = entry.get("mlp")
            if mlp is None:
                spec = None
            elif mlp.get("kind") == "dense":
                spec = MlpSpec("dense", int(mlp["ff"]))
            elif mlp.get("kind") == "moe":
                r = mlp["router"]
                spec = MlpSpec("moe", int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]))
                if spec.top < 1 or spec.top > spec.experts:
                    raise ValueError(f"layer {i}: router.top does not fit the number of experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(LayerSpec(kind, mixer, spec))
        return LamosunConfig(int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), float(d.get("postln_alpha", 1.0)),
                             float((d.get("embedding") or {}).get("scale", 1.0)),
                             int((d.get("token_side") or {}).get("dim", 0)), float(d.get("logit_softcap") or 0.0),
                             layers, d.get("architecture", "Lamosun"), d)

    @staticmethod
    def from_json(path: str) -> "LamosunConfig":
        with open(path) as f:
            return LamosunConfig.from_dict(json.load(f))


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


def addmm_f32(bias: torch.Tensor, a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """bias (fp32) + a [T, K] x w [N, K]^T with an fp32 result."""
    if a.dtype == torch.float32:
        return torch.addmm(bias, a, w.t())
    return torch.addmm(bias, a, w.t(), out_dtype=torch.float32)


class LamosunLayer(nn.Module):

    def __init__(self, cfg: LamosunConfig, index: int, spec: LayerSpec, dtype, device):
        super().__init__()
        self.spec, self.dtype, self.eps, self.alpha, W = spec, dtype, cfg.eps, cfg.alpha, cfg.width

        def vec(n=W):
            return nn.Parameter(torch.ones(n, dtype=torch.float32, device=device), requires_grad=False)

        def mat(rows, cols, dt=dtype):
            return nn.Parameter(torch.zeros((rows, cols), dtype=dt, device=device), requires_grad=False)

        self.norm1 = vec()
        m = spec.mixer
        if spec.type == "delta":
            self.conv_channels = 2 * m.kv_heads * m.dim + m.heads * m.vdim
            self.conv = ShortConv(self.conv_channels, m.taps, False, "silu", device)
            self.rule = GatedDeltaRule(m.heads, m.kv_heads, m.dim, m.vdim, cfg.eps, device)
            self.in_names = ["mix.q", "mix.k", "mix.v", "mix.g", "mix.b", "mix.a"]
            self.in_widths = [m.kv_heads * m.dim, m.kv_heads * m.dim, m.heads * m.vdim, m.heads * m.vdim, m.heads,
                              m.heads]
            self.mixed = m.heads * m.vdim
        elif spec.type == "rglru":
            self.conv = ShortConv(m.width, m.taps, True, "none", device)
            self.lru = RealGatedLRU(m.width, m.blocks, 8.0, device)
            self.in_names = ["mix.y", "mix.x"]
            self.in_widths = [m.width, m.width]
            self.mixed = m.width
        else:
            self.attn = LatentKVAttention(m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, m.rot_dims,
                                          m.rot_base, m.rot_scaling, cfg.eps, dtype, device)
            self.q_norm = vec(m.q_rank)
            self.w_uq = mat(m.heads * (m.dim + m.rot_dim), m.q_rank)
            self.in_names = ["mix.dq", "mix.dkv"]
            # the query latent's rows are padded so that the key-value part starts 16-byte aligned
            self.in_widths = [m.q_rank, m.kv_rank + m.rot_dim]
            self.q_pad = _pad8(m.q_rank) - m.q_rank
            self.mixed = m.heads * m.vdim
        # the merged input projection's rows are padded to a multiple of 8 so that every row of its
        # result starts 16-byte aligned
        rows = sum(self.in_widths) + getattr(self, "q_pad", 0)
        self.pad = _pad8(rows) - rows
        self.w_in = mat(rows + self.pad, W)
        self.b_in = nn.Parameter(torch.zeros(rows + self.pad, dtype=torch.float32, device=device),
                                 requires_grad=False) if spec.type == "rglru" else None
        self.w_out = mat(W, self.mixed)
        mlp = spec.mlp
        if mlp is not None:
            self.norm2 = vec()
            if mlp.kind == "dense":
                self.w_gate_up, self.w_down = mat(2 * mlp.ff, W), mat(W, mlp.ff)
                self.act = GatedActivation("gelu_tanh")
            else:
                self.experts = RoutedExperts(W, mlp.experts, 0, mlp.top, mlp.ff, 0, "silu", dtype=dtype, device=device,
                                             gated=True, router_bias=True)
        self.side = TokenGatedInput(W, cfg.side_dim, index * cfg.side_dim, cfg.eps, "gelu_tanh", dtype, device) \
            if cfg.side_dim else None

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self, cfg: LamosunConfig) -> Dict[str, Tuple[int, ...]]:
        """Checkpoint names (without the layer prefix) and shapes of this layer's tensors."""
        W, m, mlp = cfg.width, self.spec.mixer, self.spec.mlp
        t: Dict[str, Tuple[int, ...]] = {"norm1": (W, )}
        for name, n in zip(self.in_names, self.in_widths):
            t[name] = (n, W)
        t["mix.o"] = (W, self.mixed)
        if self.spec.type == "delta":
            for nm, n in zip(("q", "k", "v"), self.in_widths[:3]):
                t[f"mix.{nm}.conv"] = (n, m.taps)
            t.update({"mix.A_log": (m.heads, ), "mix.dt_bias": (m.heads, ), "mix.norm": (m.vdim, )})
        elif self.spec.type == "rglru":
            bw = m.width // m.blocks
            t.update({"mix.y.b": (m.width, ), "mix.x.b": (m.width, ), "mix.conv": (m.width, m.taps),
                      "mix.conv.b": (m.width, ), "mix.ra": (m.blocks, bw, bw), "mix.ra.b": (m.blocks, bw),
                      "mix.ri": (m.blocks, bw, bw), "mix.ri.b": (m.blocks, bw), "mix.lam": (m.width, )})
        else:
            t.update({"mix.dq.norm": (m.q_rank, ), "mix.uq": (m.heads * (m.dim + m.rot_dim), m.q_rank),
                      "mix.dkv.norm": (m.kv_rank, ), "mix.uk": (m.heads * m.dim, m.kv_rank),
                      "mix.uv": (m.heads * m.vdim, m.kv_rank)})
        if mlp is not None:
            t["norm2"] = (W, )
            if mlp.kind == "dense":
                t.update({"mlp.gate": (mlp.ff, W), "mlp.up": (mlp.ff, W), "mlp.down": (W, mlp.ff)})
            else:
                for e in range(mlp.experts):
                    t.update({f"mlp.e{e}.gate": (mlp.ff, W), f"mlp.e{e}.up": (mlp.ff, W), f"mlp.e{e}.down": (W, mlp.ff)})
                t["mlp.router"], t["mlp.router.b"] = (mlp.experts, W), (mlp.experts, )
        if self.side is not None:
            t.update({"side.gate": (cfg.side_dim, W), "side.proj": (W, cfg.side_dim), "side.norm": (W, )})
        return t

    def set_weights(self, t: Dict[str, torch.Tensor], cfg: LamosunConfig) -> None:
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

        self.norm1.data = f32("norm1")
        parts = [t[n].to(dt) for n in self.in_names]
        if self.spec.type == "latent_attention":
            parts.insert(1, torch.zeros((self.q_pad, W), dtype=dt))
        put(self.w_in, torch.cat(parts + [torch.zeros((self.pad, W), dtype=dt)], 0))
        put(self.w_out, t["mix.o"])
        if self.spec.type == "delta":
            self.conv.weight.data = torch.cat([t["mix.q.conv"], t["mix.k.conv"], t["mix.v.conv"]], 0).float().to(dev).contiguous()
            self.rule.a_log.data, self.rule.dt_bias.data = f32("mix.A_log"), f32("mix.dt_bias")
            self.rule.norm_weight.data = f32("mix.norm")
        elif self.spec.type == "rglru":
            self.b_in.data = torch.cat([t["mix.y.b"].float(), t["mix.x.b"].float(),
                                        torch.zeros(self.pad)], 0).to(dev).contiguous()
            self.conv.weight.data, self.conv.bias.data = f32("mix.conv"), f32("mix.conv.b")
            self.lru.set_weights(t["mix.ra"], t["mix.ra.b"], t["mix.ri"], t["mix.ri.b"], t["mix.lam"])
        else:
            self.q_norm.data = f32("mix.dq.norm")
            put(self.w_uq, t["mix.uq"])
            self.attn.set_weights(t["mix.uk"], t["mix.uv"], t["mix.dkv.norm"])
        mlp = self.spec.mlp
        if mlp is not None:
            self.norm2.data = f32("norm2")
            if mlp.kind == "dense":
                put(self.w_gate_up, torch.cat([t["mlp.gate"], t["mlp.up"]], 0))
                put(self.w_down, t["mlp.down"])
            else:
                self.experts.set_weights({k[4:]: v for k, v in t.items() if k.startswith("mlp.")})
        if self.side is not None:
            put(self.side.gate, t["side.gate"])
            put(self.side.proj, t["side.proj"])
            self.side.weight.data = f32("side.norm")

    # ------------------------------------------------------------------ caches
    def cache_shapes(self, cfg: LamosunConfig, num_blocks: int, block_size: int, num_slots: int):
        """name -> (shape, dtype) of what this layer keeps between steps."""
        m = self.spec.mixer
        out = {}
        if self.spec.type == "delta":
            if m.taps > 1:
                out["conv"] = (ShortConv.get_state_shape(num_slots, self.conv_channels, m.taps), torch.float32)
            out["state"] = (GatedDeltaRule.get_state_shape(num_slots, m.heads, m.dim, m.vdim), torch.float32)
        elif self.spec.type == "rglru":
            if m.taps > 1:
                out["conv"] = (ShortConv.get_state_shape(num_slots, m.width, m.taps), torch.float32)
            out["state"] = (RealGatedLRU.get_state_shape(num_slots, m.width), torch.float32)
        else:
            out["latent"] = (LatentKVAttention.get_cache_shape(num_blocks, block_size, m.kv_rank, m.rot_dim), self.dtype)
        return out

    # ------------------------------------------------------------------ forward
    def _mix(self, h: torch.Tensor, batch: SequenceBatch, cache: Dict[str, torch.Tensor]) -> torch.Tensor:
        T, dev, m = h.shape[0], h.device, self.spec.mixer
        if self.spec.type == "delta":
            proj = mm_f32(h, self.w_in.data)
            qkv = torch.empty((T, self.conv_channels), dtype=torch.float32, device=dev)
            self.conv(qkv, proj[:, :self.conv_channels], cache.get("conv"), batch)
            q, k, v = qkv.split(self.in_widths[:3], dim=1)
            gate, beta, dtp = proj[:, self.conv_channels:].split(self.in_widths[3:] + [self.pad], dim=1)[:3]
            mixed = torch.empty((T, self.mixed), dtype=self.dtype, device=dev)
            self.rule(mixed, q, k, v, gate, beta, dtp, cache["state"], batch)
        elif self.spec.type == "rglru":
            proj = addmm_f32(self.b_in.data, h, self.w_in.data)
            u = torch.empty((T, m.width), dtype=torch.float32, device=dev)
            self.conv(u, proj[:, m.width:2 * m.width], cache.get("conv"), batch)
            mixed = torch.empty((T, self.mixed), dtype=self.dtype, device=dev)
            self.lru(mixed, u, proj[:, :m.width], cache["state"], batch)
        else:
            proj = torch.mm(h, self.w_in.data.t())
            cq = torch.empty((T, m.q_rank), dtype=self.dtype, device=dev)
            ops.rms_norm_rows(cq, proj[:, :m.q_rank], self.q_norm.data, self.eps)
            q = torch.mm(cq, self.w_uq.data.t())
            first = m.q_rank + self.q_pad
            mixed = self.attn(q, proj[:, first:first + m.kv_rank + m.rot_dim], cache["latent"], batch)
        return mm_f32(mixed, self.w_out.data)

    def forward(self, x: torch.Tensor, h: torch.Tensor, batch: SequenceBatch, cache: Dict[str, torch.Tensor],
                side_table: Optional[torch.Tensor], input_ids: torch.Tensor) -> None:
        """x: fp32 [T, width], h: the same rows in the activation dtype; both updated in place."""
        ops.post_norm(x, self._mix(h, batch, cache), self.norm1.data, self.alpha, self.eps, h)
        mlp = self.spec.mlp
        if mlp is not None:
            if mlp.kind == "dense":
                y = mm_f32(self.act(torch.mm(h, self.w_gate_up.data.t())), self.w_down.data)
            else:
                y = self.experts(h)
            ops.post_norm(x, y, self.norm2.data, self.alpha, self.eps, h)
        if self.side is not None:
            self.side(x, h, side_table, input_ids)


class LamosunForCausalLM(nn.Module):
    """The stack and its per-layer caches.  `seed` fills random weights (benchmarks); load_weights
    installs a checkpoint's."""

    architecture = "Lamosun"

    def __init__(self, cfg: LamosunConfig, dtype=torch.bfloat16, device="cuda", seed: Optional[int] = None):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        W, L = cfg.width, len(cfg.layers)
        self.embed = nn.Parameter(torch.zeros((cfg.vocab, W), dtype=dtype, device=device), requires_grad=False)
        self.side_embed = nn.Parameter(torch.zeros((cfg.vocab, L * cfg.side_dim), dtype=dtype, device=device),
                                       requires_grad=False) if cfg.side_dim else None
        self.layers = nn.ModuleList([LamosunLayer(cfg, i, s, dtype, device) for i, s in enumerate(cfg.layers)])
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32, device=device), requires_grad=False)
        self.head = nn.Parameter(torch.zeros((cfg.vocab, W), dtype=dtype, device=device), requires_grad=False)
        if seed is not None:
            self.load_weights(self.random_weights(seed))

    # ------------------------------------------------------------------ caches
    def cache_spec(self) -> List[Dict[str, Tuple[int, ...]]]:
        """Per layer: the shapes of its caches for one block of one token and one slot."""
        return [{k: v[0] for k, v in layer.cache_shapes(self.cfg, 1, 1, 1).items()} for layer in self.layers]

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int):
        dev = self.head.device
        return [{name: torch.zeros(shape, dtype=dt, device=dev)
                 for name, (shape, dt) in layer.cache_shapes(self.cfg, num_blocks, block_size, num_slots).items()}
                for layer in self.layers]

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, caches, batch: SequenceBatch,
                tap=None) -> torch.Tensor:
        """Returns the fp32 stream [T, width] after the last layer.  tap(layer, x) is called after
        every layer (tests, layer-by-layer comparison)."""
        cfg = self.cfg
        dev = self.head.device
        x = torch.empty((input_ids.numel(), cfg.width), dtype=torch.float32, device=dev)
        ops.embed_scaled(x, self.embed.data, input_ids, cfg.embed_scale)
        h = torch.empty((input_ids.numel(), cfg.width), dtype=self.dtype, device=dev)
        ops.residual_norms(x, out=h)
        side = None if self.side_embed is None else self.side_embed.data
        for i, layer in enumerate(self.layers):
            layer(x, h, batch, caches[i], side, input_ids)
            if tap is not None:
                tap(i, x)
        return x

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """hidden: the rows of the stream whose logits are wanted -> fp32 [n, vocab]."""
        x = hidden.contiguous()
        h = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        ops.residual_norms(x, out=h, pre_weight=self.final_norm.data, eps=self.cfg.eps)
        logits = mm_f32(h, self.head.data)
        if self.cfg.softcap > 0:
            ops.softcap(logits, self.cfg.softcap)
        return logits

    # ------------------------------------------------------------------ weights
    def tensor_shapes(self) -> Dict[str, Tuple[int, ...]]:
        cfg = self.cfg
        t = {"embed": (cfg.vocab, cfg.width), "head": (cfg.vocab, cfg.width), "final.norm": (cfg.width, )}
        if cfg.side_dim:
            t["side.embed"] = (cfg.vocab, len(cfg.layers) * cfg.side_dim)
        for i, layer in enumerate(self.layers):
            t.update({f"l{i}.{k}": v for k, v in layer.tensor_shapes(cfg).items()})
        return t

    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> int:
        cfg, dev = self.cfg, self.head.device
        used = 0
        for i, layer in enumerate(self.layers):
            prefix = f"l{i}."
            mine = {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
            layer.set_weights(mine, cfg)
            used += len(layer.tensor_shapes(cfg))
        top = {"embed": (cfg.vocab, cfg.width), "head": (cfg.vocab, cfg.width), "final.norm": (cfg.width, )}
        if cfg.side_dim:
            top["side.embed"] = (cfg.vocab, len(cfg.layers) * cfg.side_dim)
        for name, shape in top.items():
            if name not in tensors:
                raise KeyError(f"tensor {name} is missing")
            if tuple(tensors[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(tensors[name].shape)}, expected {shape}")
        self.embed.data = tensors["embed"].to(self.dtype).to(dev).contiguous()
        self.head.data = tensors["head"].to(self.dtype).to(dev).contiguous()
        self.final_norm.data = tensors["final.norm"].float().to(dev).contiguous()
        if cfg.side_dim:
            self.side_embed.data = tensors["side.embed"].to(self.dtype).to(dev).contiguous()
        return used + len(top)

    def random_weights(self, seed: int) -> Dict[str, torch.Tensor]:
        """Tensors of every checkpoint name: projections ~ N(0, 1 / fan_in), norm weights near 1,
        small biases, convolution taps and decay parameters of moderate size."""
        g = torch.Generator().manual_seed(seed)
        out = {}
        for name, shape in self.tensor_shapes().items():
            last = name.rsplit(".", 1)[-1]
            if name in ("embed", "side.embed"):
                t = torch.randn(shape, generator=g)
            elif "norm" in last:
                t = 1.0 + 0.1 * torch.randn(shape, generator=g)
            elif last == "conv":
                t = 0.5 * torch.randn(shape, generator=g)
            elif len(shape) == 1 or last == "b" and len(shape) == 2 and not name.endswith("mix.b"):
                t = 0.3 * torch.randn(shape, generator=g)
            else:
                t = torch.randn(shape, generator=g) * shape[-1]**-0.5
            out[name] = t.to(torch.bfloat16)
        return out
