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
    # working from the forward's sign codes, the backward reads no entity row for the derivative
    assert bench.backward_bytes(cfg, u, from_codes=True) == back - 4 * de * u
    # the two halves of the call: ids that occur once are finished by the query-gradient kernel
    u1 = 606000
    q, e = bench.backward_kernel_bytes(cfg, u, u1, True)
    assert q == 24 * de * u1 + 4 * p + 8 * cfg["b"] * cfg["dim"] * 2 and e == 24 * de * (u - u1) + 4 * (p - u1)
    assert q + e == bench.backward_bytes(cfg, u, from_codes=True) + 4 * (p - u1)
    q, e = bench.backward_kernel_bytes(bench.CONFIGS[3], 1000, 900, False)      # rotate: rows re-read, merged rows written
    assert q == 4 * 1000 * 1000 + 4 * 1000 * 900 + 4 * 1024 * 1024 + 8 * 1024 * 500 * 2 and e == 4 * 1000 * 100 + 4 * (1024 * 1024 - 900)


def test_measured_traffic_is_tied_to_the_kernel_sources(tmp_path, monkeypatch):
    """bench.py quotes PMC traffic only from a summary taken with the kernel sources of this tree."""
    sys.path.insert(0, str(ROOT))
    import bench
    digest = bench.kernel_source_digest()
    assert len(digest) == 16 and digest == bench.kernel_source_digest()
    monkeypatch.setattr(bench, "PROFILES", str(tmp_path))
    assert bench.measured_traffic("w") is None
    rec = {"sources": digest, "commit": "abc", "kernels": {"k": [1.0, 2.0]}}
    (tmp_path / "pmc_traffic_w.md").write_text("# text\n\ntraffic_json: " + json.dumps(rec) + "\n")
    assert bench.measured_traffic("w") == rec
    rec["sources"] = "0" * 16
    (tmp_path / "pmc_traffic_w.md").write_text("traffic_json: " + json.dumps(rec) + "\n")
    assert bench.measured_traffic("w") is None


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
