"""Install shim.  pyproject.toml holds the metadata; a setuptools that reads its [project] table
(61 or newer) needs nothing else.  An older one gets the same values from here."""
from pathlib import Path

import setuptools

if int(setuptools.__version__.split('.')[0]) >= 61:
    setuptools.setup()
else:
    try:
        import tomllib as toml
    except ImportError:
        import tomli as toml
    table = toml.loads((Path(__file__).parent / 'pyproject.toml').read_text())
    project, tool = table['project'], table['tool']['setuptools']
    setuptools.setup(
        name=project['name'], version=project['version'], description=project['description'],
        python_requires=project['requires-python'], install_requires=project['dependencies'],
        extras_require=project['optional-dependencies'],
        packages=tool['packages'], package_dir=tool['package-dir'], package_data=tool['package-data'],
        entry_points={'console_scripts': [f'{name} = {target}' for name, target in project['scripts'].items()]})
