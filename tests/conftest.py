import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Writes the tiny random-weight model folders once per session; {name: path}."""
    from tiny_configs import CONFIGS
    from dinfer_amd.config.qwen3 import Qwen3Config
    from dinfer_amd.weights import write_random_model
    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        d = tmp_path_factory.mktemp(f"model_{name}")
        write_random_model(Qwen3Config.from_dict(cfg), d, seed=seed, dtype="bfloat16")
        out[name] = d
    return out
