"""torpor_amd: MI355X-native model-swapping inference server (hot path of FCSLab/torpor)."""
from .server import Server  # noqa: F401
