"""Child process of test_gpu_c_abi.py::test_fit_after_device_reset. cudaresetdevice
(src/gpu/utils.cu:40-55 in the reference's surface) frees every allocation on the device,
the library's pinned upload buffers included; a fit large enough to take the staged upload
must work before and after it and give the same result. Not collected by pytest."""
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from h2o4gpu_amd.libs import ch2o4gpu_gpu as shim  # noqa: E402

rng = np.random.default_rng(11)
n, d, k = 1_200_000, 32, 16          # 154 MB of float32: above the staging threshold
X = (rng.integers(0, k, size=n)[:, None] * 3.0 + rng.standard_normal((n, d))).astype(np.float32)
C0 = np.ascontiguousarray(X[:k])


def fit():
    pc, pl = np.zeros(k * d, np.float32), np.zeros(n, np.int32)
    rc = shim.make_ptr_float_kmeans(0, 0, 1, 0, 1, n, d, k, 5, 2, 0.0, X.reshape(-1), C0.reshape(-1), pc, pl)
    return int(rc), pc, pl


rc1, c1, l1 = fit()
reset_rc = shim.cudaresetdevice(0, 1)
rc2, c2, l2 = fit()
bare_rc = shim.cudaresetdevice_bare()
rc3, c3, l3 = fit()
print(json.dumps({"rc": [rc1, rc2, rc3], "reset_rc": [int(reset_rc), int(bare_rc)],
                  "same_centroids": bool(np.array_equal(c1, c2) and np.array_equal(c1, c3)),
                  "same_labels": bool(np.array_equal(l1, l2) and np.array_equal(l1, l3))}), flush=True)
