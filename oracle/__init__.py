"""CPU oracle for the k-means path: test infrastructure only.

Importable from tests/, the smoke check and the benchmark's CPU-baseline leg.
The engine package never imports this.
"""
from .binding import Oracle, load_oracle  # noqa: F401
