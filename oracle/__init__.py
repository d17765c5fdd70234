"""CPU oracle for the distance-neuron hot path -- TEST INFRASTRUCTURE ONLY.

Importable from tests/, the smoke check and the cpu_baseline leg of the benchmark; the
shipped package never imports it.
"""
from .oracle import *  # noqa: F401,F403
