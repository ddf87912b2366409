import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X and the built HIP library")


@pytest.fixture(scope="session")
def tiny_configs():
    """Two tiny configurations that differ in every size and option."""
    from qwen3_runtime_amd.config.presets import PRESET_PAGE_SIZE, preset

    return {name: (preset(name), PRESET_PAGE_SIZE[name]) for name in ("tiny_a", "tiny_b")}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory, tiny_configs):
    """Random-weight model folders of the tiny configurations, in a temporary place."""
    from qwen3_runtime_amd.weights import write_model_folder

    out = {}
    for i, (name, (cfg, _)) in enumerate(tiny_configs.items()):
        folder = tmp_path_factory.mktemp(name)
        write_model_folder(folder, cfg.to_dict(), seed=11 + i)
        out[name] = folder
    return out
