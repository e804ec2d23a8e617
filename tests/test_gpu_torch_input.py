"""Device-resident input (PyTorch-ROCm tensors) through the estimator."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.timeout(900)
def test_device_tensors_give_the_results_of_host_arrays(hip):
    """Runs in a child process so that PyTorch's copy of the HIP runtime is loaded
    before the engine there and never into this process (a first import of torch on a
    fresh machine can take minutes, hence the long limit)."""
    import importlib.util
    if importlib.util.find_spec("torch") is None:   # (looked up, not imported, see above)
        pytest.skip("PyTorch is not installed")
    proc = subprocess.run([sys.executable, os.path.join(HERE, "torch_device_input_check.py")],
                          capture_output=True, text=True, timeout=850)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-4000:]
    r = json.loads(proc.stdout.strip().splitlines()[-1])
    for tag in ("float32", "float64"):
        for key in ("labels_equal", "predict_equal", "transform_is_tensor", "random_close",
                    "k-means++_close", "restarts_close"):
            assert r["%s_%s" % (tag, key)] is True, (tag, key, r)
        # float32 sums are exact in double and repeat bit for bit; float64 sums depend on
        # the arrival order of the LDS adds and repeat to rounding only
        exact = tag == "float32"
        assert r[tag + "_centroids_maxdiff"] <= (0.0 if exact else 1e-13), r
        assert r[tag + "_transform_shape"] == [4096, 12]
        assert r[tag + "_n_iter"] == [7, 7]
        for key in ("_inertia", "_score"):
            a, b = r[tag + key]
            assert abs(a - b) <= (0.0 if exact else 1e-12 * abs(a)), (tag, key, r)
        if exact:
            assert r[tag + "_transform_equal"] is True, r
    assert r["strided_refused"] and r["cpu_tensor_ok"]
    assert len(r["unaligned"]) == 14
    for case, (labels_equal, diff, predict_equal) in r["unaligned"].items():
        # sums of float64 rows and of the tiled/bucketed float32 paths repeat to rounding only
        assert labels_equal and predict_equal and diff <= 1e-6, (case, r["unaligned"][case])
