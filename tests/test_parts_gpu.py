"""Each part alone on the GPU against the plain function of the same formula."""
import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu
TOL = {torch.float32: dict(atol=3e-6, rtol=3e-5), torch.bfloat16: dict(atol=0.02, rtol=0.02)}
DTYPES = [torch.float32, torch.bfloat16]


def fill(part, seed, dtype):
    """Random tensors for a part, returned as float32 CPU copies keyed by local name."""
    from qil_amd.weights.random_init import random_tensor
    from qil_amd.weights.loader import placement_dtype
    values = {}
    for name, spec in part.param_specs().items():
        t = random_tensor(spec, seed, name).to(torch.bfloat16).float()          # representable in both precisions
        values[name] = t
        part.set_param(name, t.to(placement_dtype(spec, dtype)).cuda().contiguous())
    part.finalize()
    return values


def close(actual, expected, dtype, scale=1.0):
    tol = dict(TOL[dtype], atol=TOL[dtype]['atol'] * scale)
    torch.testing.assert_close(actual.float().cpu(), expected.float(), **tol)


@pytest.mark.parametrize('dtype', DTYPES)
def test_rmsnorm_part(dtype):
    from qil_amd.parts import RMSNorm
    norm = RMSNorm(136, 3e-5)
    w = fill(norm, 1, dtype)['weight']
    stream = torch.randn(6, 136) * 2
    delta = torch.randn(6, 136).to(dtype)
    on_gpu = stream.cuda()
    out = norm.forward(on_gpu, delta.cuda(), dtype)
    summed = stream + delta.float()
    close(on_gpu, summed, torch.float32)                                       # the stream took the sum, in float32
    close(out, plain.rms_norm(summed, w, 3e-5), dtype, scale=3)
    rows = torch.tensor([4, 1], dtype=torch.int32).cuda()
    close(norm.forward_rows(on_gpu, None, rows, dtype), plain.rms_norm(summed[[4, 1]], w, 3e-5), dtype, scale=3)


def test_rotary_part_tables():
    from qil_amd.parts import Rotary
    rotary = Rotary(128, 1e6, 2048, device='cuda')
    rotation = rotary.rotation()
    angles = plain.rotary_angles(torch.arange(2048), 128, 1e6)
    assert rotation.cos.dtype == torch.float32 and rotation.rot_dim == 128
    torch.testing.assert_close(rotation.cos.cpu(), angles.cos(), atol=0, rtol=0)     # the CPU float32 table, bit for bit
    torch.testing.assert_close(rotation.sin.cpu(), angles.sin(), atol=0, rtol=0)
    # rounded to bfloat16 the table differs from the theta**(-e) variant (tests/qil/test_bf16.py:62-65)
    other = torch.arange(2048).float()[:, None] * (1e6 ** (-torch.arange(0, 128, 2, dtype=torch.float32) / 128))[None]
    assert not torch.equal(other.cos().bfloat16(), rotation.cos.cpu().bfloat16())
    partial = Rotary(64, 1e4, 16, rot_dim=32, device='cuda').rotation()
    assert partial.cos.shape == (16, 16) and partial.rot_dim == 32


@pytest.mark.parametrize('dtype', DTYPES)
def test_embedding_and_head_parts(dtype):
    from qil_amd.parts import Embedding, LMHead
    embedding, tied = Embedding(301, 72), None
    table = fill(embedding, 2, dtype)['weight']
    tokens = torch.tensor([0, 300, 7, 7], dtype=torch.int32).cuda()
    stream = embedding.forward(tokens)
    assert stream.dtype == torch.float32
    close(stream, table[tokens.cpu().long()], torch.float32)
    head = LMHead(301, 72, tied_to=embedding)
    assert head.param_specs() == {}
    rows = torch.randn(3, 72).to(dtype)
    logits = head.forward(rows.cuda())
    assert logits.dtype == torch.float32 and logits.shape == (3, 301)
    close(logits, rows.float() @ table.T, dtype, scale=0.2 if dtype == torch.bfloat16 else 3)


@pytest.mark.parametrize('dtype', DTYPES)
def test_gated_mlp_part(dtype):
    from qil_amd.parts import GatedMLP
    from qil_amd import ops
    mlp = GatedMLP(width=96, intermediate=224, dtype=dtype)
    w = fill(mlp, 3, dtype)
    for rows in (5, 40):                                                       # few rows: partial sums; many: library product
        x = torch.randn(rows, 96).to(dtype)
        out = mlp.forward(x.cuda())
        out = out.sum() if isinstance(out, ops.Partials) else out
        expected = plain.gated_mlp(x.float(), w['gate_proj.weight'], w['up_proj.weight'], w['down_proj.weight'])
        close(out, expected, dtype, scale=0.05 if dtype == torch.bfloat16 else 1)
    with pytest.raises(ValueError):
        GatedMLP(width=8, intermediate=8, activation='gelu')


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('bias', [False, True])
def test_attention_part_and_block(dtype, bias):
    """The attention part and the whole pre-norm block over a two-request batch cut into two steps,
    against plain.attention_block / plain.decoder_layer on the whole sequences."""
    from qil_amd.cache import CacheManager
    from qil_amd.engine.batch import StepContext
    from qil_amd.parts import Attention, GatedMLP, PreNormBlock, RMSNorm, Rotary
    config = dict(plain.TINY_C, attention_bias=bias, num_hidden_layers=1)
    H, nq, nkv, d = 72, 5, 1, 48
    rotary = Rotary(d, config['rope_theta'], 640, device='cuda')
    block = PreNormBlock(
        mixer_norm=RMSNorm(H, 3e-6),
        mixer=Attention(width=H, heads=nq, kv_heads=nkv, head_dim=d, bias=bias, qk_norm_eps=3e-6, scale=d ** -0.5,
                        position=rotary, dtype=dtype),
        ffn_norm=RMSNorm(H, 3e-6), ffn=GatedMLP(width=H, intermediate=136, dtype=dtype), dtype=dtype,
        names=dict(mixer_norm='input_layernorm', mixer='self_attn', ffn_norm='post_attention_layernorm', ffn='mlp'))
    weights = {}
    for prefix, part in block.parts().items():
        for local, value in fill(part, 7, dtype).items():
            weights[f'model.layers.0.{prefix}.{local}'] = value
    cache = CacheManager([block.mixer.cache_need()], num_pages=8, page_size=4, max_requests=2, dtype=dtype, device='cuda')
    for g in cache.kv_groups:
        g['k'].fill_(float('nan')), g['v'].fill_(float('nan'))
    view = cache.views()[0]
    lengths = {'a': 13, 'b': 6}
    x = {r: torch.randn(n, H).to(torch.bfloat16).float() for r, n in lengths.items()}
    streams = {r: [] for r in lengths}
    for cut in ((7, 5), (6, 1)):                                               # second step: a portion beside one token
        rows, positions, row_seq, cu, starts, slots, tables = [], [], [], [0], [], [], []
        for s, (r, size) in enumerate(zip('ab', cut)):
            start = cache.computed.get(r)
            if start is None:
                cache.admit(r)
                start = 0
            cache.ensure(r, start + size)
            rows.append(x[r][start:start + size])
            positions += list(range(start, start + size))
            row_seq += [s] * size
            cu.append(cu[-1] + size)
            starts.append(start)
            table = cache.table(0, r)
            tables.append(table + [0] * (4 - len(table)))
            slots += [table[p // 4] * 4 + p % 4 for p in range(start, start + size)]
        dev = lambda v: torch.tensor(v, dtype=torch.int32).cuda()
        single = [cu[i] for i in range(2) if cut[i] == 1]
        ctx = StepContext(n_tokens=cu[-1], n_seqs=2, n_logit_rows=0, token_ids=None, positions=dev(positions),
                          row_seq=dev(row_seq), cu_seqlens=dev(cu), seq_starts=dev(starts), seq_slots=dev([0, 1]),
                          logit_rows=None, single_rows=dev(single) if max(cut) > 1 else None, max_query=max(cut),
                          max_context=max(positions) + 1)
        view.block_tables, view.slots = dev(tables), dev(slots)
        stream = torch.cat(rows).cuda()
        pending = block.forward(stream, None, ctx, view)
        from qil_amd import ops
        pending = pending.sum() if isinstance(pending, ops.Partials) else pending
        total = stream + pending.float()
        at = 0
        for r, size in zip('ab', cut):
            streams[r].append(total[at:at + size])
            at += size
            cache.advance(r, cache.computed[r] + size)
    for r, n in lengths.items():
        expected = plain.decoder_layer(x[r], weights, 0, config, torch.arange(n))
        close(torch.cat(streams[r]), expected, dtype, scale=0.5 if dtype == torch.bfloat16 else 2)
