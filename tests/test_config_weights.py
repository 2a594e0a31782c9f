"""Configuration, registry and weight loading (CPU)."""
import json

import pytest
import torch
from safetensors.torch import save_file

import plain_qwen3 as plain
from conftest import write_model_folder
from qil_amd.config import ConfigError, Qwen3Config
from qil_amd.registry import known_architectures, read_model_config, architecture_for
from qil_amd.weights import WeightsError, load_model, write_random_model


def test_registry_names_and_reads():
    assert known_architectures() == ['Qwen3ForCausalLM']
    entry = architecture_for(dict(plain.TINY_B))
    assert entry.config_class is Qwen3Config
    without_name = {k: v for k, v in plain.TINY_B.items() if k != 'architectures'}
    assert architecture_for(without_name).name == 'Qwen3ForCausalLM'             # falls back on model_type
    with pytest.raises(ConfigError, match='unknown architecture'):
        architecture_for(dict(plain.TINY_B, architectures=['LlamaForCausalLM']))


def test_config_fields_defaults_and_rejections(tmp_path):
    config = Qwen3Config.from_dict(plain.TINY_B)
    assert (config.hidden_size, config.head_dim, config.rms_norm_eps, config.rope_theta) == (96, 32, 1e-5, 1e6)
    assert config.eos_ids == frozenset({7, 9}) and not config.tie_word_embeddings
    minimal = {k: plain.TINY_A[k] for k in ('model_type', 'vocab_size', 'hidden_size', 'intermediate_size',
                                            'num_hidden_layers', 'num_attention_heads', 'num_key_value_heads',
                                            'head_dim', 'max_position_embeddings')}
    defaults = Qwen3Config.from_dict(minimal)                                     # qil/config.py:18-22
    assert (defaults.rms_norm_eps, defaults.rope_theta, defaults.attention_bias, defaults.tie_word_embeddings,
            defaults.eos_token_id) == (1e-6, 1e6, False, True, None)
    assert Qwen3Config.from_dict(defaults.to_dict()) == defaults
    assert defaults.torch_dtype is None                                          # informational: kept, never acted on
    assert Qwen3Config.from_dict(dict(minimal, torch_dtype='bfloat16')).to_dict()['torch_dtype'] == 'bfloat16'
    for patch in (dict(model_type='qwen3_moe'), dict(rope_scaling={'rope_type': 'linear'}),      # tests/qil/test_model.py:72-80
                  dict(use_sliding_window=True), dict(hidden_act='gelu'), dict(layer_types=['sliding_attention']),
                  dict(vocab_size=0), dict(head_dim=15), dict(num_key_value_heads=3), dict(rms_norm_eps=0.0),
                  dict(rope_theta=float('inf')), dict(hidden_size=64.0), dict(attention_bias='no'), dict(torch_dtype=16)):
        with pytest.raises(ConfigError):
            Qwen3Config.from_dict(dict(plain.TINY_A, **patch))
    with pytest.raises(ConfigError, match='required'):
        Qwen3Config.from_dict({k: v for k, v in plain.TINY_A.items() if k != 'head_dim'})
    with pytest.raises(ConfigError, match='config.json'):
        read_model_config(tmp_path)
    (tmp_path / 'config.json').write_text(json.dumps(plain.TINY_A))
    entry, config = read_model_config(tmp_path)
    assert entry.name == 'Qwen3ForCausalLM' and config.vocab_size == 256


@pytest.mark.parametrize('config', [plain.TINY_A, plain.TINY_B, plain.TINY_C])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_load_places_every_tensor(tmp_path, config, dtype):
    weights = plain.random_weights(config, 5)
    write_model_folder(tmp_path, config, weights, torch.bfloat16)
    model = load_model(tmp_path, dtype=dtype, device='cpu')
    assert model.loaded and model.dtype == dtype
    assert set(model.names) == set(plain.tensor_shapes(config))                  # same names as qil/model.py:159-176
    attention = model.blocks[0].mixer
    q = config['num_attention_heads'] * config['head_dim']
    torch.testing.assert_close(attention.w_qkv[:q].float(), weights['model.layers.0.self_attn.q_proj.weight'])
    assert attention.w_qkv.dtype == dtype                                         # matrices in the model's dtype
    assert model.final_norm.p['weight'].dtype == torch.float32                    # vectors stay float32
    torch.testing.assert_close(model.final_norm.p['weight'], weights['model.norm.weight'])
    if config['tie_word_embeddings']:
        assert model.head.weight is model.embedding.p['weight']
    if config['attention_bias']:
        assert attention.b_qkv.shape == (q + 2 * config['num_key_value_heads'] * config['head_dim'],)
    gate_up = model.blocks[1].ffn.p['gate_up_proj.weight']
    torch.testing.assert_close(gate_up[config['intermediate_size']:].float(), weights['model.layers.1.mlp.up_proj.weight'])


def test_sharded_folder_and_tied_names(tmp_path):
    config, weights = plain.TINY_A, plain.random_weights(plain.TINY_A, 2)
    names = sorted(weights)
    (tmp_path / 'config.json').write_text(json.dumps(config))
    save_file({n: weights[n] for n in names[::2]}, str(tmp_path / 'model-00001-of-00002.safetensors'))
    second = {n: weights[n] for n in names[1::2]}
    second['lm_head.weight'] = weights['model.embed_tokens.weight'].clone()      # both names of a tied tensor, equal
    save_file(second, str(tmp_path / 'model-00002-of-00002.safetensors'))
    model = load_model(tmp_path, dtype=torch.float32, device='cpu')
    torch.testing.assert_close(model.head.weight, weights['model.embed_tokens.weight'])


def corrupt(weights, how):
    weights = {k: v.clone() for k, v in weights.items()}
    if how == 'missing':
        del weights['model.norm.weight'], weights['model.layers.1.mlp.up_proj.weight']
    elif how == 'shape':
        weights['model.norm.weight'] = torch.ones(1)
    elif how == 'extra':
        weights['unknown.weight'] = torch.ones(1)
    elif how == 'tied':
        weights['lm_head.weight'] = weights['model.embed_tokens.weight'] + 1
    elif how == 'type':
        weights['model.norm.weight'] = weights['model.norm.weight'].to(torch.int32)
    return weights


@pytest.mark.parametrize('how', ['missing', 'shape', 'extra', 'tied', 'type'])          # tests/qil/test_model.py:54-69
def test_corrupt_checkpoints_fail_with_one_clear_error(tmp_path, how):
    (tmp_path / 'config.json').write_text(json.dumps(plain.TINY_A))
    save_file(corrupt(plain.random_weights(plain.TINY_A, 0), how), str(tmp_path / 'model.safetensors'))
    with pytest.raises(WeightsError) as error:
        load_model(tmp_path, dtype=torch.float32, device='cpu')
    text = str(error.value)
    word = dict(missing='missing tensors', shape='wrong shapes', extra='unexpected tensors', tied='inconsistent tied',
                type='wrong element types')[how]
    assert word in text
    if how == 'missing':
        assert 'model.norm.weight' in text and 'model.layers.1.mlp.up_proj.weight' in text


def test_all_faults_are_listed_together(tmp_path):
    weights = corrupt(corrupt(corrupt(plain.random_weights(plain.TINY_A, 0), 'missing'), 'extra'), 'shape')
    weights['model.norm.weight'] = torch.ones(3)
    write_model_folder(tmp_path, plain.TINY_A, weights)
    with pytest.raises(WeightsError) as error:
        load_model(tmp_path, dtype=torch.float32, device='cpu')
    text = str(error.value)
    assert all(word in text for word in ('missing tensors', 'unexpected tensors', 'wrong shapes', 'unknown.weight'))


def test_no_weight_files(tmp_path):
    (tmp_path / 'config.json').write_text(json.dumps(plain.TINY_A))
    with pytest.raises(WeightsError, match='safetensors'):
        load_model(tmp_path, dtype=torch.float32, device='cpu')


def test_random_model_folder(tmp_path):
    a = write_random_model(tmp_path / 'a', plain.TINY_B, seed=7)
    b = write_random_model(tmp_path / 'b', Qwen3Config.from_dict(plain.TINY_B), seed=7)
    c = write_random_model(tmp_path / 'c', plain.TINY_B, seed=8)
    assert sorted(p.name for p in a.iterdir()) == ['config.json', 'model.safetensors']
    ma, mb, mc = (load_model(p, dtype=torch.float32, device='cpu') for p in (a, b, c))
    wa, wb, wc = (m.blocks[2].mixer.w_qkv for m in (ma, mb, mc))
    torch.testing.assert_close(wa, wb, atol=0, rtol=0)                            # the seed fixes the weights
    assert not torch.equal(wa, wc)
    assert 0.015 < wa.std() < 0.025                                               # N(0, 0.02)
    norm = ma.final_norm.p['weight']
    assert abs(norm.mean() - 1) < 0.01 and 0.005 < norm.std() < 0.015            # 1 + N(0, 0.01)
    half = load_model(a, dtype=torch.bfloat16, device='cpu')                     # stored as bfloat16: both precisions share values
    torch.testing.assert_close(half.blocks[2].mixer.w_qkv.float(), wa, atol=0, rtol=0)


def test_model_schedule_is_data(tmp_path):
    """The run order is a list: it may name a block twice or let an entry read another entry's cache."""
    from qil_amd.parts import ScheduleEntry, KVNeed
    from qil_amd.registry import architecture_for
    entry = architecture_for(plain.TINY_A)
    model = entry.build(entry.config_class.from_dict(plain.TINY_A), dtype=torch.float32, device='cpu')
    assert [e.block for e in model.schedule] == [0, 1] and all(e.cache_of is None for e in model.schedule)
    model.schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_of=1)]
    needs = model.cache_needs()
    assert needs[:3] == [KVNeed(2, 16, None)] * 3 and needs[3] == ('shared', 1)
    from qil_amd.cache import CacheManager
    cache = CacheManager(needs, num_pages=4, page_size=4, max_requests=2, allocate=True)
    assert cache.kv_groups[0]['entries'] == [0, 1, 2] and cache.kv_groups[0]['k'].shape[0] == 3
    views = cache.views()
    assert views[3].k.data_ptr() == views[1].k.data_ptr() and not views[3].writes and views[1].writes
    with pytest.raises(ValueError):
        type(model)(config=model.config, embedding=model.embedding, blocks=model.blocks,
                    schedule=[ScheduleEntry(0, cache_of=0)], final_norm=model.final_norm, head=model.head,
                    names=model.names, tied=model.tied, dtype=torch.float32, device='cpu')
