"""Device helpers used by the estimator (reference: src/interface_py/h2o4gpu/util/gpu.py)."""
