"""Packaging entry for setuptools.  All metadata lives in pyproject.toml; setuptools older than
61 does not read the [project] / [tool.setuptools] tables, so they are handed over here."""

import os

import setuptools

HERE = os.path.dirname(os.path.abspath(__file__))


def _tables():
    try:
        import tomllib as toml
    except ImportError:  # Python < 3.11
        import tomli as toml
    with open(os.path.join(HERE, "pyproject.toml"), "rb") as f:
        return toml.load(f)


def _legacy_arguments():
    doc = _tables()
    project, tool = doc["project"], doc["tool"]["setuptools"]
    return dict(
        name=project["name"],
        version=project["version"],
        description=project["description"],
        python_requires=project["requires-python"],
        install_requires=project["dependencies"],
        entry_points={group: [f"{name} = {target}" for name, target in entries.items()]
                      for group, entries in project["entry-points"].items()},
        packages=tool["packages"],
        package_dir=tool["package-dir"],
        package_data=tool["package-data"],
        include_package_data=False,
    )


if int(setuptools.__version__.split(".")[0]) < 61:
    setuptools.setup(**_legacy_arguments())
else:
    setuptools.setup()
