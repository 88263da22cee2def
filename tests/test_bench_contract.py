"""bench.py's fixed figures against the committed profile summaries, and its command line contract.  No GPU needed."""
import importlib.util
import re
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def _bench():
    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_measured_traffic_constant_matches_the_profile_summary():
    """roofline.traffic is a measured figure held as a constant in bench.py: it must be the one the committed
    rocprofv3 --pmc summary derives."""
    text = (ROOT / "profiles" / "decode_layer_b1_gemv_hbm_traffic.md").read_text()
    m = re.search(r"Average over the four launches of a layer pass:\s*([0-9,]+)\s*B", text)
    assert m, "the traffic summary no longer states the per-launch average"
    assert int(m.group(1).replace(",", "")) == _bench().MEASURED_TRAFFIC_BYTES_PER_LAUNCH


def test_layer_bytes_is_the_sum_of_the_seven_projections():
    b = _bench()
    kv = b.KV_HEADS * b.HEAD_DIM
    shapes = [(b.HIDDEN, b.HIDDEN), (kv, b.HIDDEN), (kv, b.HIDDEN), (b.HIDDEN, b.HIDDEN), (b.FFN, b.HIDDEN), (b.FFN, b.HIDDEN),
              (b.HIDDEN, b.FFN)]
    assert sum(n * k // 4 for n, k in shapes) == b.LAYER_BYTES == 17_367_040
    assert b.LAYER_BYTES * b.LAYERS == b.STEP_BYTES == 521_011_200
    assert b.LAUNCHES_PER_STEP == 4 * b.LAYERS
    assert b.REPEATS >= 5


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode != 0 and "one-GPU" in proc.stderr
