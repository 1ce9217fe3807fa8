"""CPU oracle for the MoE-MLP hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this; it is used by tests/, by __graft_entry__.smoke() and
by the cpu_baseline leg of bench.py as the checker / reported baseline, never as the product path.
"""
from .naive_moe import *  # noqa: F401,F403
