"""The package installs under the import name ``qil_amd`` with a console script (pyproject.toml), and the
uninstalled checkout imports under the same name from any directory."""
import os
import shutil
import subprocess
import sys

import pytest

from conftest import ROOT


def clean_environment(**extra):
    env = {k: v for k, v in os.environ.items() if k != 'PYTHONPATH'}
    env.update(extra)
    return env


def test_checkout_imports_from_another_directory(tmp_path):
    code = 'import qil_amd, qil_amd.engine, qil_amd.cache; print(qil_amd.__file__); print(qil_amd.Engine.__module__)'
    run = subprocess.run([sys.executable, '-c', code], cwd=tmp_path, env=clean_environment(PYTHONPATH=str(ROOT)),
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    where, module = run.stdout.split()
    assert where == str(ROOT / 'qwen-inference-lab_amd' / '__init__.py') and module == 'qil_amd.engine.engine'
    run = subprocess.run([sys.executable, '-m', 'qil_amd', '--help'], cwd=tmp_path,
                         env=clean_environment(PYTHONPATH=str(ROOT)), capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and '--token-ids' in run.stdout and '--chunk-size' in run.stdout


def test_install_and_console_script(tmp_path):
    pytest.importorskip('setuptools')
    source = tmp_path / 'source'
    source.mkdir()
    for name in ('pyproject.toml', 'setup.py', 'README.md'):
        shutil.copy(ROOT / name, source / name)
    shutil.copytree(ROOT / 'qwen-inference-lab_amd', source / 'qwen-inference-lab_amd',
                    ignore=shutil.ignore_patterns('_build', '__pycache__'))
    site = tmp_path / 'site'
    install = subprocess.run([sys.executable, '-m', 'pip', 'install', '--no-build-isolation', '--no-deps', '--no-index',
                              '--quiet', '--target', str(site), str(source)], capture_output=True, text=True, timeout=600,
                             cwd=tmp_path)
    if install.returncode != 0 and 'No module named pip' in install.stderr:
        pytest.skip('pip is not available')
    assert install.returncode == 0, install.stderr[-3000:]
    script = site / 'bin' / 'qil-amd'
    assert script.exists()
    elsewhere = tmp_path / 'elsewhere'
    elsewhere.mkdir()
    env = clean_environment(PYTHONPATH=str(site))
    run = subprocess.run([sys.executable, str(script), '--help'], cwd=elsewhere, env=env, capture_output=True, text=True,
                         timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert '--token-ids' in run.stdout and '--max-new-tokens' in run.stdout
    code = ('import qil_amd, pathlib; from qil_amd.ops import library; print(qil_amd.__file__); '
            'print(len(library.sources())); import qil_amd.engine, qil_amd.weights, qil_amd.sampling, qil_amd.models')
    run = subprocess.run([sys.executable, '-c', code], cwd=elsewhere, env=env, capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    where, count = run.stdout.split()
    assert where == str(site / 'qil_amd' / '__init__.py')
    assert int(count) == len(list((ROOT / 'qwen-inference-lab_amd' / 'csrc').glob('*.hip'))) > 0   # the HIP sources travel
