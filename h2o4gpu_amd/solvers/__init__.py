"""Estimators (reference: src/interface_py/h2o4gpu/solvers)."""
from .kmeans import KMeans, KMeansH2O  # noqa: F401
