"""Grouped-query attention over the paged cache.  Formulas: qil/model.py:48-69, :73-84."""
import torch

from .base import Mixer, ParamSpec, KVNeed
from .. import ops


class Attention(Mixer):
    """q/k/v projections (+bias), optional per-head RMSNorm of q and k, position
    encoding, write of k/v into the request's pages, attention of the step's
    queries over everything cached (key j visible iff j <= position, and
    j > position - window if a window is set), output projection (+bias).

    Query head h reads kv head h // (heads / kv_heads)  (qil/model.py:59-61).
    The three projection matrices are stacked at ``finalize`` into one
    [(heads + 2 kv_heads) head_dim, width] matrix: a pure re-layout, each output
    column is computed from the same row as before.
    """
    graph_safe = True
    takes_lazy_norm = True       # h goes into ops.linear only, which takes a norm not computed yet

    def __init__(self, *, width, heads, kv_heads, head_dim, bias, qk_norm_eps, scale,
                 position=None, window=None, dtype=torch.bfloat16):
        super().__init__()
        if heads % kv_heads:
            raise ValueError('heads must be a multiple of kv_heads')
        self.width, self.heads, self.kv_heads, self.head_dim = width, heads, kv_heads, head_dim
        self.bias, self.qk_norm_eps, self.scale = bool(bias), qk_norm_eps, float(scale)
        self.position, self.window, self.dtype = position, window, dtype
        ops.check_attention_geometry(heads=heads, kv_heads=kv_heads, head_dim=head_dim, dtype=dtype)

    def param_specs(self):
        q, kv, d = self.heads * self.head_dim, self.kv_heads * self.head_dim, self.head_dim
        specs = {'q_proj.weight': ParamSpec((q, self.width)), 'k_proj.weight': ParamSpec((kv, self.width)),
                 'v_proj.weight': ParamSpec((kv, self.width)), 'o_proj.weight': ParamSpec((self.width, q))}
        if self.bias:   # o_proj gets a bias too (qil/model.py:35)
            specs.update({'q_proj.bias': ParamSpec((q,), 'vector'), 'k_proj.bias': ParamSpec((kv,), 'vector'),
                          'v_proj.bias': ParamSpec((kv,), 'vector'), 'o_proj.bias': ParamSpec((self.width,), 'vector')})
        if self.qk_norm_eps is not None:
            specs.update({'q_norm.weight': ParamSpec((d,), 'vector', 'one_plus_normal'),
                          'k_norm.weight': ParamSpec((d,), 'vector', 'one_plus_normal')})
        return specs

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window)

    def finalize(self):
        p = self.p
        self.w_qkv = torch.cat([p.pop('q_proj.weight'), p.pop('k_proj.weight'), p.pop('v_proj.weight')]).contiguous()
        self.b_qkv = (torch.cat([p.pop('q_proj.bias'), p.pop('k_proj.bias'), p.pop('v_proj.bias')]).contiguous()
                      if self.bias else None)
        p['qkv_proj.weight'] = self.w_qkv
        if self.bias:
            p['qkv_proj.bias'] = self.b_qkv

    def forward(self, h, ctx, cache):
        p = self.p
        qkv = ops.linear(h, self.w_qkv, self.b_qkv, partials=True)
        rotation = self.position.rotation() if self.position is not None else None
        norms = dict(q_weight=p.get('q_norm.weight'), k_weight=p.get('k_norm.weight'),
                     eps=self.qk_norm_eps if self.qk_norm_eps is not None else 0.0)
        sizes = dict(heads=self.heads, kv_heads=self.kv_heads, head_dim=self.head_dim)
        if ctx.max_query == 1 and ops.decode_attention_takes(qkv, page_size=cache.page_size, rotation=rotation,
                                                             dtype=self.dtype, **sizes):
            # every row alone in its sequence: norm, rotation and cache write happen inside the attention kernel
            attended = ops.decode_attention(
                qkv, rotation=rotation, positions=ctx.positions, writes=cache.writes, k_cache=cache.k, v_cache=cache.v,
                page_size=cache.page_size, block_tables=cache.block_tables, row_seq=ctx.row_seq,
                max_context=ctx.max_context, scale=self.scale, window=self.window, unmerged=True, **sizes, **norms)
            return ops.linear(attended, p['o_proj.weight'], p.get('o_proj.bias'), partials=True)
        q = ops.qk_norm_rope_store(
            qkv, rotation=rotation, positions=ctx.positions, slots=cache.slots if cache.writes else None,
            k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size, dtype=self.dtype, **sizes, **norms)
        attended = ops.paged_attention(
            q, k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size,
            block_tables=cache.block_tables, row_seq=ctx.row_seq, positions=ctx.positions,
            cu_seqlens=ctx.cu_seqlens, seq_starts=ctx.seq_starts, single_rows=ctx.single_rows, n_seqs=ctx.n_seqs,
            max_query=ctx.max_query, max_context=ctx.max_context, tile_seqs=ctx.tile_seqs,
            scale=self.scale, window=self.window, unmerged=True, **sizes)
        return ops.linear(attended, p['o_proj.weight'], p.get('o_proj.bias'), partials=True)
