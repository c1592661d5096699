"""Causal softmax attention whose keys and values are up-projections of one cached latent.

Per token the layer caches one row [c | k_rot]: the RMS-normed latent c (`rank` numbers) and a
rotated key part (`rot` numbers) that all heads share -- cache [num_blocks, block_size, rank + rot].
Head h scores a query (q_plain [dim], q_rot [rot]) against key j as
(q_plain . W_uk,h c_j + q_rot . k_rot_j) * scale and sums values W_uv,h c_j.  Both up-projections
are moved to the query's side, where they cost one batched matrix product per step each:
q_lat,h = W_uk,h^T q_plain,h scores the cached latent directly, and the head's output is
W_uv,h (sum_j p_j c_j).  Rotation: pairs (2i, 2i + 1) when `interleaved`, (i, i + rot_dims / 2)
otherwise, of the first `rot_dims` elements of the rotated parts turn by position * f_i, sine and
cosine times `magnitude` (a frequency table and a magnitude as YaRN scaling gives them, or plain
ones).  `scale` multiplies the scores as it is.  An optional `window` keeps 0 <= i - j < window;
an optional gate [T, heads] multiplies each head's output by its sigmoid (applied to the latent
sums, ahead of the linear up-projection).  Prompts, portions of prompts and decode steps are one case: the step's rows are written to
the cache, then every query row reads from there (csrc/seq_latent_attention.hip: a matrix-core
kernel for 16-bit models whose rank is a multiple of 32 and whose rotated part is a multiple of 16,
and an fp32 kernel for any dtype and size).
"""
import math
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from vllm_legacy_amd import _seq_ops as ops
from vllm_legacy_amd.attention.batch import SequenceBatch


def yarn_frequencies(dims: int, base: float, scaling: Optional[Dict] = None,
                     device=None) -> Tuple[torch.Tensor, float]:
    """(f_i fp32 [dims / 2], magnitude).  Without scaling f_i = base^(-2i / dims) and the magnitude
    is 1.  With scaling {factor, original, fast, slow}: a pair that makes `t` turns over `original`
    positions sits at d(t) = dims ln(original / (2 pi t)) / (2 ln base); pairs below
    lo = floor(d(fast)) keep their frequency, pairs above hi = ceil(d(slow)) get f_i / factor, a
    linear ramp joins them, and sine and cosine are multiplied by 0.1 ln(factor) + 1.  Formed in
    float64, rounded once to fp32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / float(dims))
    magnitude = 1.0
    if scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def place(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(place(float(scaling["fast"]))), 0)
        hi = min(math.ceil(place(float(scaling["slow"]))), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        magnitude = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32).to(device), magnitude


class LatentKVAttention(nn.Module):

    def __init__(self, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, rank: int, scale: float,
                 rot_dims: int, rot_base: float, rot_scaling: Optional[Dict], eps: float, dtype=torch.bfloat16,
                 device=None, interleaved: bool = True, window: Optional[int] = None) -> None:
        super().__init__()
        assert 0 <= rot_dims <= rot_dim and rot_dims % 2 == 0
        self.interleaved, self.window = bool(interleaved), int(window) if window else 0
        self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.rank = num_heads, head_dim, rot_dim, value_dim, rank
        self.scale, self.rot_dims, self.eps, self.dtype = float(scale), int(rot_dims), float(eps), dtype
        inv_freq, self.magnitude = yarn_frequencies(rot_dims, rot_base, rot_scaling, device) if rot_dims else (None, 1.0)
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        self.latent_norm = nn.Parameter(torch.ones(rank, dtype=torch.float32, device=device), requires_grad=False)
        # W_uk as [heads, dim, rank] (q_lat = q_plain W_uk,h) and W_uv^T as [heads, rank, vdim]
        self.w_uk = nn.Parameter(torch.zeros((num_heads, head_dim, rank), dtype=dtype, device=device),
                                 requires_grad=False)
        self.w_uv_t = nn.Parameter(torch.zeros((num_heads, rank, value_dim), dtype=dtype, device=device),
                                   requires_grad=False)

    def set_weights(self, uk: torch.Tensor, uv: torch.Tensor, latent_norm: torch.Tensor) -> None:
        """uk [heads * dim, rank], uv [heads * vdim, rank] (rows head by head), latent_norm [rank]."""
        dev = self.w_uk.device
        H, D, V, C = self.num_heads, self.head_dim, self.value_dim, self.rank
        self.w_uk.data = uk.to(self.dtype).view(H, D, C).to(dev).contiguous()
        self.w_uv_t.data = uv.to(self.dtype).view(H, V, C).transpose(1, 2).to(dev).contiguous()
        self.latent_norm.data = latent_norm.float().to(dev).contiguous()

    # workgroups a launch should have before the keys of a row tile stay with one workgroup
    SPLIT_BELOW_WORKGROUPS = 512
    KEYS_PER_SPLIT = 256

    def key_splits(self, batch: SequenceBatch) -> int:
        """Steps of few rows over long contexts (decode steps) share every row tile's keys out to
        several workgroups: enough of them to fill the part, none with fewer than KEYS_PER_SPLIT
        keys."""
        heads_per = min(self.num_heads, 32)
        tiles = -(-batch.max_query_len // (32 // heads_per)) * -(-self.num_heads // heads_per) * batch.num_seqs
        if tiles >= self.SPLIT_BELOW_WORKGROUPS:
            return 1
        keys = batch.max_seq_len
        if self.window:
            keys = min(keys, self.window + batch.max_query_len)
        return max(1, min(-(-self.SPLIT_BELOW_WORKGROUPS // tiles), keys // self.KEYS_PER_SPLIT, 32))

    @staticmethod
    def get_cache_shape(num_blocks: int, block_size: int, rank: int, rot_dim: int) -> Tuple[int, ...]:
        return (num_blocks, block_size, rank + rot_dim)

    def forward(self, q: torch.Tensor, kv: torch.Tensor, cache: torch.Tensor, batch: SequenceBatch,
                gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q [T, heads * (dim + rot_dim)], head by head [plain | rotated] (rotated in place); kv
        [T, rank + rot_dim] before its norm and rotation, gate [T, heads] (views with free row
        strides).  Returns [T, heads * vdim]."""
        T = q.shape[0]
        H, D, Rr, V, C = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.rank
        ops.latent_rotary_write(q, D + Rr, D, H, kv, self.latent_norm.data, self.eps, cache, batch.positions,
                                batch.slot_mapping, self.inv_freq, self.magnitude, self.rot_dims, self.interleaved)
        q3 = q.view(T, H, D + Rr)
        q_lat = torch.bmm(q3[:, :, :D].transpose(0, 1), self.w_uk.data)             # [H, T, C]
        o_lat = torch.empty((H, T, C), dtype=q.dtype, device=q.device)
        q_lat, q_rot, o_rows = q_lat.transpose(0, 1), q3[:, :, D:], o_lat.transpose(0, 1)
        if ops.latent_attention_tiles_supported(q_lat, q_rot, cache):
            # 16-bit models whose sizes fit: (token, head) rows in tiles of 32 on the matrix cores
            ops.latent_attention_tiles(o_rows, q_lat, q_rot, cache, batch.block_tables, batch.query_start_loc,
                                       batch.context_lens, batch.max_query_len, self.scale,
                                       self.key_splits(batch), self.window, gate)
        else:
            ops.latent_attention(o_rows, q_lat, q_rot, cache, batch.block_tables, batch.token_seq, batch.positions,
                                 self.scale, self.window, gate)
        o = torch.bmm(o_lat, self.w_uv_t.data)                                      # [H, T, V]
        return o.transpose(0, 1).reshape(T, H * V)
