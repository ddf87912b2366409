import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X and the built HIP library")


def pytest_terminal_summary(terminalreporter):
    """With -v: how far the bfloat16 comparisons of the run stayed below their bounds."""
    import traces

    if traces.MEASURED_NOISE and terminalreporter.config.option.verbose > 0:
        terminalreporter.write_line(f"bfloat16 against plain, {len(traces.MEASURED_NOISE)} comparisons; the largest "
                                    f"rms and the largest error, in units of the logits' deviation:")
        for rms, worst, test in sorted(traces.MEASURED_NOISE, reverse=True)[:5]:
            terminalreporter.write_line(f"  rms {rms:.4f} worst {worst:.4f} {test}")


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
