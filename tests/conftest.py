import json
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
for path in (str(ROOT), str(ROOT / 'tests')):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs an MI355X (run with -m gpu on the GPU box)')


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason='no GPU here')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def cpu_kernels(monkeypatch):
    """Run the engine's host logic on the CPU by substituting the kernels' plain references."""
    import kernel_refs
    from qil_amd import ops
    for name, function in kernel_refs.ALL.items():
        monkeypatch.setattr(ops, name, function)
    return kernel_refs


def write_model_folder(directory, config, weights, dtype=torch.float32):
    """config.json + model.safetensors from the plain implementation's weights."""
    from safetensors.torch import save_file
    directory = Path(directory)
    directory.mkdir(parents=True, exist_ok=True)
    (directory / 'config.json').write_text(json.dumps(config))
    save_file({name: t.to(dtype).contiguous() for name, t in weights.items()}, str(directory / 'model.safetensors'))
    return directory


@pytest.fixture
def model_folder(tmp_path):
    def make(config, seed, dtype=torch.float32, **kwargs):
        import plain_qwen3 as plain
        weights = plain.random_weights(config, seed, **kwargs)
        folder = write_model_folder(tmp_path / f'model{seed}_{abs(hash(json.dumps(config, sort_keys=True))) % 10**8}',
                                    config, weights, dtype)
        return folder, weights
    return make
