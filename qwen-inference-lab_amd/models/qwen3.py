"""Dense Qwen3 assembled from parts.

Architecture as the reference runs it (qil/model.py:26-40, :89-104): token
embedding; per layer RMSNorm -> grouped-query attention with per-head RMSNorm of
q and k, full-width rotary encoding and scale head_dim**-0.5 -> add; RMSNorm ->
SiLU-gated MLP -> add; final RMSNorm; head, tied to the embedding on request.
Tensor names: qil/model.py:159-176.
"""
import torch

from ..config.qwen3 import Qwen3Config
from ..parts import (RMSNorm, Rotary, Attention, GatedMLP, PreNormBlock, Embedding, LMHead,
                     CausalLM, ScheduleEntry)
from ..registry import register_architecture


def _full_attention(config, rotary, dtype):
    return Attention(width=config.hidden_size, heads=config.num_attention_heads,
                     kv_heads=config.num_key_value_heads, head_dim=config.head_dim,
                     bias=config.attention_bias, qk_norm_eps=config.rms_norm_eps,
                     scale=config.head_dim ** -0.5, position=rotary, window=None, dtype=dtype)


def _dense_mlp(config, dtype):
    return GatedMLP(width=config.hidden_size, intermediate=config.intermediate_size, activation='silu', dtype=dtype)


# Layer kinds this architecture can hold, chosen layer by layer.
MIXERS = {'full_attention': _full_attention}
FEED_FORWARDS = {'dense': _dense_mlp}

_BLOCK_NAMES = dict(mixer_norm='input_layernorm', mixer='self_attn',
                    ffn_norm='post_attention_layernorm', ffn='mlp')


def layer_plan(config):
    """(mixer kind, feed-forward kind) of every layer; uniform for dense Qwen3."""
    return [('full_attention', 'dense')] * config.num_hidden_layers


def build_qwen3(config, *, dtype=torch.bfloat16, device='cuda'):
    rotary = Rotary(config.head_dim, config.rope_theta, config.max_position_embeddings, device=device)
    embedding = Embedding(config.vocab_size, config.hidden_size)
    blocks = []
    for mixer_kind, ffn_kind in layer_plan(config):
        blocks.append(PreNormBlock(
            mixer_norm=RMSNorm(config.hidden_size, config.rms_norm_eps),
            mixer=MIXERS[mixer_kind](config, rotary, dtype),
            ffn_norm=RMSNorm(config.hidden_size, config.rms_norm_eps),
            ffn=FEED_FORWARDS[ffn_kind](config, dtype), dtype=dtype, names=_BLOCK_NAMES))
    final_norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
    head = LMHead(config.vocab_size, config.hidden_size,
                  tied_to=embedding if config.tie_word_embeddings else None)

    names = {'model.embed_tokens.weight': (embedding, 'weight'), 'model.norm.weight': (final_norm, 'weight')}
    for index, block in enumerate(blocks):
        for prefix, part in block.parts().items():
            for local in part.param_specs():
                names[f'model.layers.{index}.{prefix}.{local}'] = (part, local)
    tied = {}
    if config.tie_word_embeddings:
        tied['lm_head.weight'] = 'model.embed_tokens.weight'
    else:
        names['lm_head.weight'] = (head, 'weight')
    return CausalLM(config=config, embedding=embedding, blocks=blocks,
                    schedule=[ScheduleEntry(i) for i in range(len(blocks))],
                    final_norm=final_norm, head=head, names=names, tied=tied, dtype=dtype, device=device)


register_architecture('Qwen3ForCausalLM', model_type='qwen3', config_class=Qwen3Config, build=build_qwen3,
                      replace=True)
