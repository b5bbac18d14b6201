"""Latent attention: keys and values of all heads are products of one cached vector per token.

Per token, with h the mixer's input:  q = W_q h, head by head [nope_dim unrotated | rope_dim rotated];
W_down h has kv_rank + rope_dim rows: the first kv_rank, RMS-normed with a weight, are the latent c,
the last rope_dim are one key part shared by all heads.  Head j's key is [W_uk_j c | shared part], its
value W_uv_j c; query and shared key part are rotated by position; the score is

    (q_nope . W_uk_j c + q_rot . k_rot) * scale

over the keys the mask lets through (a sliding window, chunks, or every earlier key), an ordinary
softmax, and W_o on the concatenated heads.

For designs that have them: a learned sink per head that joins the softmax's denominator as exp(sink), without
a key or a value and not scaled (`sinks`); no rotated part at all (`rope_dim` 0); and layers without a down
projection that read the rows an earlier layer cached, with their own W_uk, W_uv, queries and mask (`own_kv` False:
the stop borrows that layer's pages).

What the cache holds of a token is c and the rotated part, one row of kv_rank + rope_dim whatever the number
of heads (`paged_spec`: one tensor "latent" [PAGE][kv_rank + rope_dim]).  The heads' keys and values
are never formed: since q_nope . (W_uk_j c) = (W_uk_j^T q_nope) . c, the query is folded into latent
space once per token ([W_uk_j^T q_nope | q_rot], kv_rank + rope_dim wide), the attention kernel scores
it against the cached row as it is and sums the rows' first kv_rank features as values, and the
head's output is W_uv_j times that sum.  The query projection and the down projection are one
product; the two per-head products are one launch each.
"""

from __future__ import annotations

import torch

from ..cache.manager import PAGE, PagedSpec, PagedTensor
from ..kernels import lib as K
from .base import POSITION_ENCODINGS, Part, ScaleShape, StepShape, build_part, plain_rows, register_mixer
from .linear import Linear, rows_a_graph_may_hold


def latent_pages(kv_rank: int, rope_dim: int, window=None, transposed: bool = False) -> PagedSpec:
    """One row per token: the latent vector, then the rotated key part.  `transposed`: also the latents
    transposed within the page, [kv_rank][PAGE], the layout the matrix-core kernel reads its values in."""
    tensors = (PagedTensor("latent", (PAGE, kv_rank + rope_dim)),)
    if transposed:
        tensors += (PagedTensor("latent_t", (kv_rank, PAGE)),)
    return PagedSpec(tensors, window)


def latent_tiles(shape: StepShape, single: int, runs: int):
    """Work lists of the matrix-core kernel: (table row, first flat token, tokens, 0) for every sequence that
    brings one token (`single`), and for the others in pieces of up to `runs` tokens, those with the most keys first."""
    one, many = [], []
    for row, (start, n, past) in enumerate(zip(shape.q_starts, shape.q_lens, shape.past_lens)):
        if n == 1:
            one += [row, start, 1, 0]
        else:
            for first in range(0, n, runs):
                many.append((past + first, (row, start + first, min(runs, n - first), 0)))
    many.sort(key=lambda piece: -piece[0])
    return {"single": (one, 4), "runs": ([x for _, piece in many for x in piece], 4)}


@register_mixer("latent_attention")
class LatentAttention(Part):
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if min(spec.num_heads, spec.nope_dim, spec.value_dim, spec.kv_rank) <= 0 or spec.rope_dim < 0:
            raise ValueError("latent attention: heads, nope_dim, value_dim and kv_rank must be positive")
        if spec.kv_rank + spec.rope_dim > 1024 or spec.kv_rank > 512:
            raise ValueError(f"latent attention: kv_rank {spec.kv_rank} + rope_dim {spec.rope_dim}: the kernels take "
                             "rows up to 1024 with a latent up to 512")
        if spec.mask not in ("window", "chunk"):
            raise ValueError(f"mask '{spec.mask}' is not known (known: window, chunk)")
        if spec.mask == "chunk" and not spec.window:
            raise ValueError("a mask in chunks needs the chunk length (window)")
        if not spec.own_kv and spec.rope_dim:
            raise ValueError("a latent layer that reads another layer's rows has no rotated part")
        rotated = getattr(spec.position, "rotary_dim", 0) if spec.position is not None else 0
        if rotated > spec.rope_dim:
            raise ValueError(f"{rotated} rotated features of a rotated part of {spec.rope_dim}")
        self.position = (build_part(POSITION_ENCODINGS, "position encoding", spec.position, dtype, device)
                         if spec.position is not None else POSITION_ENCODINGS["none"](None, dtype, device))
        if not hasattr(self.position, "rotary_table") or float(getattr(self.position, "magnitude", 1.0)) != 1.0:
            raise ValueError("latent attention rotates by a plain table of cosines and sines")

    @property
    def graph_safe(self) -> bool:
        return self.position.graph_safe

    @property
    def graph_max_rows(self):
        s = self.spec
        return rows_a_graph_may_hold(self.dtype, s.hidden_size, s.num_heads * s.value_dim)

    @property
    def row_width(self) -> int:
        return self.spec.kv_rank + self.spec.rope_dim

    @property
    def matrix_cores(self) -> bool:
        """Whether the attention runs on the matrix cores (then the pages also hold the latents transposed)."""
        return K.latent_attn_supported(self.dtype, self.row_width, self.spec.kv_rank)

    def paged_spec(self):
        s = self.spec
        return latent_pages(s.kv_rank, s.rope_dim, s.window if s.mask == "window" else None, self.matrix_cores)

    def step_lists_key(self, block_size: int):
        if not (self.matrix_cores and block_size % 16 == 0):
            return None
        H = self.spec.num_heads
        return ("latent attention tiles", K.latent_attn_tokens(H, 1), K.latent_attn_tokens(H, 2))

    def step_lists(self, shape: StepShape):
        H = self.spec.num_heads
        return latent_tiles(shape, K.latent_attn_tokens(H, 1), K.latent_attn_tokens(H, 2))

    def tensors(self, prefix):
        s = self.spec
        sfx = s.weight_suffix
        out = {prefix + s.q_name + sfx: (s.num_heads * (s.nope_dim + s.rope_dim), s.hidden_size),
               prefix + s.up_k_name + sfx: (s.num_heads * s.nope_dim, s.kv_rank),
               prefix + s.up_v_name + sfx: (s.num_heads * s.value_dim, s.kv_rank),
               prefix + s.o_name + sfx: (s.hidden_size, s.num_heads * s.value_dim)}
        if s.own_kv:
            out[prefix + s.down_name + sfx] = (self.row_width, s.hidden_size)
            out[prefix + s.down_norm_name] = ScaleShape((s.kv_rank,))
        if s.sinks:
            out[prefix + s.sink_name] = (s.num_heads,)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        sfx = s.weight_suffix
        projected = [weights[prefix + s.q_name + sfx]] + ([weights[prefix + s.down_name + sfx]] if s.own_kv else [])
        self.proj = Linear(self.matrix(torch.cat(projected, dim=0)))
        self.down_norm = self.vector(weights[prefix + s.down_norm_name]) if s.own_kv else None
        # sinks enter the softmax, which is float32
        self.sinks = (weights[prefix + s.sink_name].to(device=self.device, dtype=torch.float32).contiguous()
                      if s.sinks else None)
        up_k = weights[prefix + s.up_k_name + sfx].view(s.num_heads, s.nope_dim, s.kv_rank)
        # the fold q_nope -> W_uk^T q_nope is a product with W_uk^T as its [out, in] matrix, head by head
        self.up_k_t = self.matrix(up_k.transpose(1, 2))
        self.up_v = self.matrix(weights[prefix + s.up_v_name + sfx].view(s.num_heads, s.value_dim, s.kv_rank))
        self.out = Linear(self.matrix(weights[prefix + s.o_name + sfx]))

    def forward(self, ctx, x):
        s = self.spec
        if s.own_kv != ctx.writes_cache:
            raise ValueError("a latent layer with a down projection writes its own pages, one without reads another stop's")
        x = plain_rows(x)
        T, H, C, R, D, V = x.shape[0], s.num_heads, s.kv_rank, s.rope_dim, s.nope_dim, s.value_dim
        pages = ctx.cache.pages_of(ctx.cache_entry)
        latent, latent_t = pages["latent"], pages.get("latent_t")
        table = ctx.block_tables[ctx.cache.group_of(ctx.cache_entry)]
        proj = self.proj(x)
        rot, cos_sin = self.position.rotary_table(ctx)
        q_full = torch.empty((T, H * (C + R)), dtype=proj.dtype, device=proj.device)
        if s.own_kv:
            K.latent_prepare(proj, q_full, H, D, R, rot, bool(getattr(self.position, "interleaved", False)), C,
                             self.down_norm, s.norm_eps, cos_sin, ctx.positions, ctx.tok_seq, table, latent, latent_t)
        K.heads_product(q_full.view(T, H, C + R)[:, :, :C], proj[:, :H * (D + R)].view(T, H, D + R)[:, :, :D], self.up_k_t)
        summed = torch.empty((T, H * C), dtype=proj.dtype, device=proj.device)
        key = self.step_lists_key(ctx.cache.block_size)
        if key is not None and latent_t is not None:
            tiles = ctx.memo[key]
            for name, column_tiles in (("single", 1), ("runs", 2)):
                if tiles[name].numel():
                    K.latent_attn(summed, q_full, latent, latent_t, tiles[name], column_tiles, ctx.positions, table, H, C,
                                  s.scale, s.window or 0, s.mask == "chunk", self.sinks)
        else:
            K.paged_attention_masked(summed, q_full, latent, None, ctx.positions, ctx.tok_seq, table, H, 1, C + R, C, s.scale,
                                     s.window or 0, s.mask == "chunk", sinks=self.sinks)
        heads = torch.empty((T, H * V), dtype=proj.dtype, device=proj.device)
        K.heads_product(heads.view(T, H, V), summed.view(T, H, C), self.up_v)
        return self.out.branch(heads, ctx.sink)
