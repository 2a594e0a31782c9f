"""The engine runs with every other engine and model framework barred from import.

The reference holds the same guard for its own package (tests/qil/test_independence.py:6-22): a
subprocess replaces ``__import__`` with one that refuses those packages, then loads a model folder
and generates.  Here the barred list also names the packages whose model code this repository must
not lean on.
"""
import subprocess
import sys
from pathlib import Path

import pytest

import plain_qwen3 as plain

ROOT = Path(__file__).resolve().parent.parent

GUARD = '''
import builtins, sys
sys.path.insert(0, {root!r})
barred = {{'nano_vllm', 'nanovllm', 'vllm', 'transformers', 'triton', 'flash_attn', 'xformers', 'accelerate',
          'sglang', 'deepspeed'}}
original = builtins.__import__
def restricted(name, *args, **kwargs):
    if name.split('.')[0] in barred:
        raise AssertionError('barred import: ' + name)
    return original(name, *args, **kwargs)
builtins.__import__ = restricted
'''


def run(code, *args):
    subprocess.run([sys.executable, '-c', GUARD.format(root=str(ROOT)) + code, *map(str, args)], check=True, timeout=300)


def test_package_imports_without_other_engines():
    run('''
import qil_amd
from qil_amd import Engine, Qwen3
import qil_amd.cache, qil_amd.config, qil_amd.engine, qil_amd.models, qil_amd.parts, qil_amd.sampling, qil_amd.weights
import qil_amd.__main__, qil_amd.engine.replay
assert not barred & {name.split('.')[0] for name in sys.modules}, barred & set(sys.modules)
''')


@pytest.mark.gpu
def test_generation_without_other_engines(model_folder):
    folder, _ = model_folder(plain.TINY_A, 5)
    run('''
import torch
from qil_amd import Engine, Qwen3
engine = Engine(Qwen3.from_directory(sys.argv[1], device='cuda', dtype=torch.bfloat16), num_pages=8, page_size=4)
results = engine.generate([[1, 2, 3], [4, 5, 6]], max_new_tokens=3, ignore_eos=True)
assert all(len(result['token_ids']) == 3 and result['state'] == 'completed' for result in results)
engine.cache.check()
assert engine.cache.free_pages == [8]
assert not barred & {name.split('.')[0] for name in sys.modules}
''', folder)
