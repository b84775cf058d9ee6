"""MI355X-native per-batch planning path of LPLB: histogram -> LP solve -> redirect."""
from .planner import Planner
from .topology import CUBE_8P2E, HYPERCUBE_16P2E, RING_8P, torus_2d

__all__ = ["Planner", "CUBE_8P2E", "HYPERCUBE_16P2E", "RING_8P", "torus_2d"]
