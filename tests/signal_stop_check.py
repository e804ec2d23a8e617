"""Child process of test_gpu_c_abi.py::test_sigint_stops_the_loop_when_handlers_are_enabled.
With H2O4GPU_KMEANS_SIGNALS=1 the library installs the reference's SIGINT/SIGTERM handler
(kmeans_h2o4gpu.cu:581-582, kmeans_impl.h:210-215): a signal ends the Lloyd loop after the
current iteration, the final relabel still runs and the call returns 0. Not collected by
pytest."""
import json
import os
import signal
import sys
import threading
import time

import numpy as np

os.environ["H2O4GPU_KMEANS_SIGNALS"] = "1"
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from h2o4gpu_amd.libs import ch2o4gpu_gpu as shim  # noqa: E402

rng = np.random.default_rng(5)
n, d, k, max_iter = 200_000, 16, 8, 2_000_000
X = (rng.integers(0, k, size=n)[:, None] * 4.0 + rng.standard_normal((n, d))).astype(np.float32)
C0 = np.ascontiguousarray(X[:k])
pc, pl = np.zeros(k * d, np.float32), np.zeros(n, np.int32)
threading.Timer(0.4, lambda: os.kill(os.getpid(), signal.SIGINT)).start()
t0 = time.perf_counter()
rc = shim.make_ptr_float_kmeans(0, 0, 1, 0, 1, n, d, k, max_iter, 2, 0.0, X.flatten(), C0.flatten(), pc, pl)
dt = time.perf_counter() - t0
info = shim.last_fit_info()
print(json.dumps({"rc": int(rc), "seconds": dt, "iterations": info[1] if info else None,
                  "labels_in_range": bool(((pl >= 0) & (pl < k)).all())}), flush=True)
