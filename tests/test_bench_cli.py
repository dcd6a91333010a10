"""Host-side contract of bench.py and of the product path that needs no GPU."""
import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_byte_models_of_the_headline_workload():
    sys.path.insert(0, str(ROOT))
    import bench
    cfg = bench.CONFIGS[5]
    u, p, de = 748072, cfg["b"] * cfg["k"], 200
    step = bench.algorithmic_bytes(cfg, u)
    assert step == 4 * de * 2 * u + 24 * de * u + 16 * p + 12 * cfg["b"] * cfg["dim"] * 2
    back = bench.backward_bytes(cfg, u)
    assert back == 4 * de * u + 24 * de * u + 4 * p + 8 * cfg["b"] * cfg["dim"] * 2
    assert bench.algorithmic_bytes(cfg, u, streaming=True) > step


def test_product_path_has_no_cpu_fallback():
    """Without a GPU the fused entry points must raise, not compute on the host."""
    torch = pytest.importorskip("torch")
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from smore_amd import _lib, fused
    t = torch.zeros(4, 8)
    with pytest.raises(Exception):
        fused.score_forward("l1", t, torch.zeros(2, 2, dtype=torch.int64), torch.zeros(2, 8), None, fused.score_params(1.0))
    assert callable(_lib.load)


def test_committed_profiles_name_their_commands():
    for f in (ROOT / "profiles").glob("*.md"):
        text = f.read_text()
        assert "rocprofv3" in text and "bench.py" in text, f.name
